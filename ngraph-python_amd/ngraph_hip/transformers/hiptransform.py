"""`hipgpu`: the MI355X transformer for fused elementwise / reduction graphs.

Plays the part of ngraph/transformers/gputransform.py for this path:

* `kernel_op_name` maps each op class to a kernel op name the way
  `ElementWiseKernel.add_op` does (gputransform.py:124-275);
* `FusionPlanner` groups consecutive elementwise ops (optionally ended by
  reductions) that share an iteration space into one kernel spec.  The
  reference generator supports such compounds (float_ew2.py:553-612,
  1135-1429) but its transformer hands it one op at a time
  (gputransform.py:381-391); `fusion=False` reproduces that;
* operands become (pointer, element strides) views over at most three merged
  axes (float_ew2.py:289-338, MAX_AXES = 3), reductions see the reduced axes
  first (gputransform.py:117-122);
* `HipKernelGroup.__call__` is the executor loop (gputransform.py:508-522);
* `HipDeviceBufferStorage` / `HipDeviceTensor` own device memory and do host
  I/O, strided views going through the device copy kernel
  (gputransform.py:525-909).

All arithmetic runs in libngraph_hip.so; if the library or a GPU is missing,
constructing the transformer raises.
"""
from __future__ import division
from collections import OrderedDict

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.op_graph.op_graph import Op, OrderedSet
from ngraph_hip.runtime import hiplib
from ngraph_hip.runtime.hiplib import (HipRuntime, DryRunRuntime, HipLibraryError, FusedSpecBuilder, NGH_F32,
                                       NGH_FLEX16, NGH_I32, NGH_F16, NGH_U32, NGH_I16, NGH_I8, NGH_U8,
                                       NGH_MAX_TENSORS,
                                       NGH_MAX_OPS, NGH_MAX_CONSTS, NGH_MAX_REGS,
                                       NGH_MAX_REDUCTIONS, NGH_CACHE_STREAM_LOAD,
                                       NGH_CACHE_STREAM_STORE)
from ngraph_hip.transformers.base import (ComputationGraphTransformer, DeviceBufferStorage,
                                          DeviceTensor, UnsupportedTransformerException)
from ngraph_hip.transformers.passes.passes import SimplePrune, PeepholeGraphPass
from ngraph_hip.transformers.passes.hippasses import TensorSizeFold, ReductionLayoutPass, ConstantFoldPass

# op class -> kernel op name (gputransform.py:129-275)
_UNARY_NAMES = OrderedDict([
    (og.AbsoluteOp, "abs"), (og.CosOp, "cos"), (og.ExpOp, "exp"), (og.LogOp, "log"),
    (og.NegativeOp, "neg"), (og.ReciprocalOp, "rcp"), (og.SignOp, "sgn"),
    (og.SigmoidAtomicOp, "sig"), (og.SinOp, "sin"), (og.SqrtOp, "sqrt"), (og.SquareOp, "sqr"),
    (og.TanhOp, "tanh"),
])
_BINARY_NAMES = OrderedDict([
    (og.Add, "add"), (og.Divide, "div"), (og.FloorDivide, "int_div"), (og.Mod, "mod"),
    (og.Equal, "eq"), (og.Greater, "gt"), (og.GreaterEqual, "ge"), (og.Less, "lt"),
    (og.LessEqual, "le"), (og.Maximum, "maximum"), (og.Minimum, "minimum"),
    (og.Multiply, "mul"), (og.NotEqual, "ne"), (og.Power, "pow"), (og.Subtract, "sub"),
])
_REDUCTION_NAMES = OrderedDict([
    (og.Sum, "sum"), (og.Prod, "prod"), (og.Max, "max"), (og.Min, "min"),
    (og.Argmax, "argmax"), (og.Argmin, "argmin"),
])


def _td(op):
    """The tensor description of `op` in this backend's conventions: strides and offset in
    elements, one stride per axis.  The graph front of this repository describes tensors that
    way itself (`_adapt_td` is the identity); the plug-in for the real package, whose
    descriptions hold byte strides and nested strides for flattened axes
    (ngraph/op_graph/axes.py:1174-1232), replaces `_adapt_td`."""
    return _adapt_td(op.tensor_description())


def _adapt_td(td):
    return td


def _lookup(table, op):
    for cls, name in table.items():
        if isinstance(op, cls):
            return name
    return None


def kernel_op_name(op):
    """Kernel op name of a graph op, or None when it is not an elementwise/reduction op."""
    return _lookup(_UNARY_NAMES, op) or _lookup(_BINARY_NAMES, op) or _lookup(_REDUCTION_NAMES, op)


def is_fusable(op):
    return (kernel_op_name(op) is not None or
            isinstance(op, (og.AssignOp, og.OneHotOp, og.Fill, og.LookupTableOp, og.RngOp)))


def iteration_axes(op):
    """Named axes a kernel running `op` loops over."""
    if isinstance(op, og.ReductionOp):
        return op.args[0].forwarded.axes
    if isinstance(op, (og.AssignOp, og.Fill)):
        return op.args[0].forwarded.axes
    return op.axes


def _scalar_constant_value(op):
    """Python float of a scalar constant reached only through views, else None."""
    cur = op.forwarded
    while True:
        if isinstance(cur, og.AssignableTensorOp):
            if cur.is_constant and cur.is_scalar:
                return float(np.asarray(cur.const).reshape(()))
            return None
        if isinstance(cur, og.TensorValueOp):
            cur = cur.value_tensor.forwarded
        elif isinstance(cur, og.IndexOp):
            cur = cur.args[0].forwarded
        else:
            return None


def _producer(op):
    """The device op (or state tensor) whose buffer `op` is a view of."""
    cur = op.forwarded
    while True:
        if isinstance(cur, og.TensorValueOp):
            cur = cur.value_tensor.forwarded
        elif isinstance(cur, og.IndexOp):
            cur = cur.args[0].forwarded
        elif isinstance(cur, og.SequentialOp):
            cur = cur.value_tensor.forwarded
        else:
            return cur


def _memory_elements(td):
    """Distinct elements a view touches (a broadcast axis repeats the same ones)."""
    n = 1
    for length, stride in zip(td.shape, td.full_strides):
        if stride != 0:
            n *= length
    return n


def _view_key(td):
    return (td.base, td.parameter_key)


# =============================================================================== storage
class HipDeviceBufferStorage(DeviceBufferStorage):
    """One device allocation per base tensor (gputransform.py:642-676); allocated on first use."""

    def __init__(self, transformer, bytes, dtype, **kwargs):
        super(HipDeviceBufferStorage, self).__init__(transformer, bytes, dtype, **kwargs)
        self._ptr = None

    @property
    def ptr(self):
        if self._ptr is None:
            self._ptr = self.transformer.runtime.malloc(max(int(self.bytes), 4))
        return self._ptr

    def create_device_tensor(self, tensor_description):
        return HipDeviceTensor(self.transformer, self, tensor_description,
                               name="v_" + tensor_description.name)

    def free(self):
        if self._ptr is not None:
            self.transformer.runtime.free(self._ptr)
            self._ptr = None


class HipDeviceTensor(DeviceTensor):
    """A strided view of a device buffer with host I/O (gputransform.py:679-909)."""

    storage_np_dtype = None   # None: the logical dtype

    def transform_allocate(self):
        pass

    @property
    def view(self):
        """The view's description with strides and offset in elements (see _td)."""
        return _adapt_td(self.tensor_description)

    @property
    def np_dtype(self):
        d = self.tensor_description.dtype
        return d if isinstance(d, np.dtype) else np.dtype(np.int16)

    @property
    def ngh_dtype(self):
        return self.transformer.ngh_dtype(self.tensor_description.dtype)

    @property
    def itemsize(self):
        return self.np_dtype.itemsize

    @property
    def ptr(self):
        return self.device_buffer.ptr + self.view.offset * self.itemsize

    @property
    def shape(self):
        return self.view.shape

    @property
    def element_strides(self):
        return self.view.full_strides

    def _read_raw(self):
        """The view's elements as a C-contiguous host array of the storage dtype."""
        td, rt = self.view, self.transformer.runtime
        out = np.empty(td.shape, dtype=self.np_dtype)
        if out.size == 0:
            return out
        if td.c_contiguous:
            rt.memcpy_d2h(out, self.ptr)
            return out
        # strided or broadcast view: gather on the device (into the context's scratch), then one
        # contiguous copy out
        tmp = rt.io_scratch(out.nbytes)
        contiguous = [int(s) // out.itemsize for s in out.strides]
        rt.copy_strided(tmp, self.ptr, td.shape, contiguous, td.full_strides, out.itemsize)
        rt.memcpy_d2h(out, tmp)
        return out

    def _write_window(self, host, offset, shape, strides):
        """host (broadcast to `shape`) into the window of the buffer that starts `offset` elements
        into this view and has the given element strides."""
        rt = self.transformer.runtime
        host = np.ascontiguousarray(np.broadcast_to(host, shape), dtype=self.np_dtype)
        if host.size == 0:
            return
        ptr = self.ptr + offset * self.itemsize
        dense, run = True, 1
        for n, s in zip(reversed(shape), reversed(strides)):
            dense = dense and (n == 1 or s == run)
            run *= n
        if dense:
            rt.memcpy_h2d(ptr, host)
            return
        if any(s == 0 and n > 1 for s, n in zip(strides, shape)):
            raise ValueError("cannot write through a broadcast view")
        # one contiguous copy in (the host copy returns when the data has arrived), then a
        # scatter on the device, which later kernels on the stream are ordered behind
        tmp = rt.io_scratch(host.nbytes)
        rt.memcpy_h2d(tmp, host)
        contiguous = [int(s) // host.itemsize for s in host.strides]
        rt.copy_strided(ptr, tmp, shape, strides, contiguous, host.itemsize)

    def _write_raw(self, host):
        td = self.view
        self._write_window(host, 0, td.shape, td.full_strides)

    def get(self, tensor):
        value = self._read_raw()
        if tensor is None:
            return value
        tensor[...] = value
        return tensor

    def __getitem__(self, key):
        return self.get(None)[key]

    def _window_of(self, key):
        """(offset, shape, strides) in elements of view[key] for a key made of integers and
        slices (what NumPy calls basic indexing); None for anything else."""
        td = self.view
        key = key if isinstance(key, tuple) else (key,)
        if any(k is Ellipsis for k in key):
            i = [k is Ellipsis for k in key].index(True)
            if any(k is Ellipsis for k in key[i + 1:]):
                return None
            key = key[:i] + (slice(None),) * (len(td.shape) - (len(key) - 1)) + key[i + 1:]
        if len(key) > len(td.shape):
            return None
        key = key + (slice(None),) * (len(td.shape) - len(key))
        offset, shape, strides = 0, [], []
        for k, n, s in zip(key, td.shape, td.full_strides):
            if isinstance(k, (int, np.integer)):
                k = int(k)
                if not -n <= k < n:
                    raise IndexError("index %d is out of bounds for an axis of length %d" % (k, n))
                offset += (k % n) * s
            elif isinstance(k, slice):
                lo, hi, step = k.indices(n)
                count = len(range(lo, hi, step))
                offset += lo * s if count else 0
                shape.append(count)
                strides.append(s * step)
            else:
                return None
        return offset, shape, strides

    def __setitem__(self, key, value):
        value = np.asarray(value)
        if key is Ellipsis or key == () or (isinstance(key, slice) and key == slice(None, None, None)):
            self._write_raw(value.astype(self.np_dtype, copy=False))
            return
        window = self._window_of(key)
        if window is not None and all(s >= 0 for s in window[2]):
            # only the addressed window travels: a contiguous copy in and a strided copy on the device
            self._write_window(value.astype(self.np_dtype, copy=False), *window)
            return
        whole = self._read_raw()
        whole[key] = value
        self._write_raw(whole)


# =============================================================================== kernels
class HipKernel(object):
    """One launchable unit of a computation (gpu/kernel.py:18-87)."""

    def __init__(self, transformer):
        self.transformer = transformer
        self.buffers_bound = False

    def bind_buffers(self):
        self.buffers_bound = True

    def execute(self):
        raise NotImplementedError

    # flex hooks (flexgputransform.py:56-61, 347-366)
    output_flex_ids = ()
    output_flex_entries = ()

    def bind_flex_scales(self):
        pass

    def probe(self):
        pass


def _no_uses(self):
    return []


def _ignore_hints(self, hint_of):
    pass


HipKernel.buffer_uses = _no_uses
HipKernel.set_cache_hints = _ignore_hints


class _Dim(object):
    __slots__ = ("length", "strides", "tag", "named")

    def __init__(self, length, strides, tag=None, named=None):
        # tag "red" marks a reduced axis; `named` keeps the axis name of a dim some op refers
        # to by coordinate (one-hot, lookup), which therefore must not merge with another
        self.length, self.strides, self.tag, self.named = int(length), list(strides), tag, named


def _emit_program(sb, program, inner):
    """Append `program` (tuples over symbolic registers, FusedKernel._collect) to the spec builder
    as the ops of its current stage; returns the operand slots it reads and writes."""
    reg_map = {}

    def reg(sym):
        if sym not in reg_map:
            reg_map[sym] = sb.reg()
        return reg_map[sym]

    written, read = set(), set()
    for ins in program:
        kind = ins[0]
        if kind == "const":
            sb.constant(ins[2], reg(ins[1]))
        elif kind == "load":
            sb.load(ins[2], reg(ins[1]))
            read.add(ins[2])
        elif kind in ("store", "store_trunc"):
            sb.store(ins[1], reg(ins[2]), truncate=(kind == "store_trunc"))
            written.add(ins[1])
        elif kind == "iota":
            axis = [i for i, d in enumerate(inner) if d.named == ins[2].name]
            if not axis:
                raise og_unsupported("one-hot axis was merged away")
            sb.iota(axis[0], reg(ins[1]))
        elif kind == "rng":
            sb.rng(ins[2], ins[3], reg(ins[1]))
        elif kind == "take":
            axis = [i for i, d in enumerate(inner) if d.named == ins[4].name]
            if not axis:
                raise og_unsupported("lookup axis was merged away or looped on the host")
            sb.take(ins[3], reg(ins[2]), axis[0], reg(ins[1]))
            read.add(ins[3])
        elif kind == "reduce":
            sb.reduce(ins[1], reg(ins[2]), ins[3])
            written.add(ins[3])
        elif len(ins) == 3:
            sb.unary(kind, reg(ins[2]), reg(ins[1]))
        else:
            sb.binary(kind, reg(ins[2]), reg(ins[3]), reg(ins[1]))
    return read, written


class FusedKernel(HipKernel):
    """A compound elementwise / reduction kernel = one ngh_fused_spec per outer index.

    `ops` are the graph ops of the group, in execution order.  Lowering
    happens in bind_buffers, once storage exists.
    """

    def __init__(self, transformer, ops, store_ops, name):
        super(FusedKernel, self).__init__(transformer)
        self.ops = list(ops)
        self.store_ops = set(store_ops)
        self.name = name
        self.kernel_number = transformer.n_kernels      # distinguishes the random streams of kernels
        transformer.n_kernels += 1
        self.n_rng_streams = 0
        self.specs = []
        self.flex_bindings = []     # (spec index, tensor slot, flex entry, is_output)
        self.spec_uses = []         # per spec: [(base tensor description, is read, is written)] per slot
        self.described = None

    fill_store = "store"         # how a Fill writes its value (a flex kernel truncates)

    def _constant_value(self, value):
        """The fp32 immediate a scalar constant becomes (a flex kernel quantises it first)."""
        return value

    # -- operand bookkeeping ------------------------------------------------------------
    def bind_buffers(self):
        if not self.buffers_bound:
            self._lower()
        super(FusedKernel, self).bind_buffers()

    def _collect(self):
        """Pass 1 of the lowering: the operands (views) the group touches and its program over
        symbolic registers; returns (operands, program, it_axes, red_axes, onehot_axes,
        take_axes, take_strides)."""
        ops = self.ops
        reductions = [op for op in ops if isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1]
        # (a kernel may carry a few ops over a subset of its axes, absorbed from a smaller kernel:
        # they are simply repeated along the missing axes)
        it_axes = iteration_axes(max(ops, key=lambda o: (len(iteration_axes(o)), iteration_axes(o).size)))
        red_axes = reductions[0].reduction_axes if reductions else og.make_axes(())
        onehot_axes = [op.axis for op in ops if isinstance(op, og.OneHotOp)]
        take_axes = []           # output axes whose coordinate a lookup replaces by an index value
        take_strides = {}        # (operand slot, axis) -> the table's stride along its looked-up axis
        self.take_extents = {}   # operand slot -> length of the table's looked-up axis
        self.n_rng_streams = 0   # random fills in this kernel, each its own stream

        # ---- pass 1: collect operands (views) and the program over symbolic registers ----
        operands = []            # [(td, role)] in slot order
        slot_of = {}             # view key -> slot
        program = []             # tuples, see _emit below
        value_reg = {}           # producing op / view key -> symbolic register
        n_sym = [0]

        def new_reg():
            n_sym[0] += 1
            return n_sym[0] - 1

        def slot(td):
            key = _view_key(td)
            if key not in slot_of:
                slot_of[key] = len(operands)
                operands.append(td)
            return slot_of[key]

        def operand_reg(arg):
            arg = arg.forwarded
            c = _scalar_constant_value(arg)
            if c is not None:
                r = new_reg()
                program.append(("const", r, self._constant_value(c)))
                return r
            prod = _producer(arg)
            if prod in value_reg:
                return value_reg[prod]
            td = _td(arg)
            key = _view_key(td)
            if key in value_reg:
                return value_reg[key]
            r = new_reg()
            program.append(("load", r, slot(td)))
            value_reg[key] = r
            return r

        red_slots = []
        reductions_at_end = []
        for op in ops:
            name = kernel_op_name(op)
            if isinstance(op, og.AssignOp):
                target, val = op.args[0].forwarded, op.args[1].forwarded
                r = operand_reg(val)
                td = _td(target)
                program.append(("store", slot(td), r))
                value_reg[_view_key(td)] = r
                continue
            if isinstance(op, og.Fill):
                td = _td(op.args[0].forwarded)
                r = new_reg()
                program.append(("const", r, float(op.scalar)))
                program.append((self.fill_store, slot(td), r))
                value_reg[_view_key(td)] = r
                continue
            if isinstance(op, og.OneHotOp):
                x = operand_reg(op.args[0])
                i = new_reg()
                program.append(("iota", i, op.axis))
                r = new_reg()
                program.append(("eq", r, i, x))
            elif isinstance(op, og.RngOp):
                # RngFillKernel (tensor_ops.py:651-661): draw, then scale and shift
                u = new_reg()
                program.append(("rng", u, op.distribution, self.n_rng_streams))
                self.n_rng_streams += 1
                if op.distribution == "uniform":
                    mul, add = op.params["high"] - op.params["low"], op.params["low"]
                else:
                    mul, add = op.params["scale"], op.params["loc"]
                c_mul, c_add, m, r = new_reg(), new_reg(), new_reg(), new_reg()
                program.append(("const", c_mul, float(mul)))
                program.append(("mul", m, u, c_mul))
                program.append(("const", c_add, float(add)))
                program.append(("add", r, m, c_add))
            elif isinstance(op, og.LookupTableOp):
                # gputransform.py:197-199: ("take", x=idx, y=lut, axis=lut_axis)
                lut, idx = op.args[0].forwarded, op.args[1].forwarded
                x = operand_reg(idx)
                lut_td = _td(lut)
                table = slot(lut_td)
                out_axis = op.axes[op.lut_axis]
                take_axes.append(out_axis)
                take_strides[(table, out_axis)] = lut_td.full_strides[op.lut_axis]
                self.take_extents[table] = lut_td.shape[op.lut_axis]
                r = new_reg()
                program.append(("take", r, x, table, out_axis))
            elif isinstance(op, og.ReductionOp):
                x = operand_reg(op.args[0])
                if len(op.reduction_axes) == 0 or op.reduction_axes.size == 1:
                    # nothing to reduce: assign (gputransform.py:117-119, float_ew2.py:582-586)
                    r = new_reg()
                    if name in ("argmax", "argmin"):
                        program.append(("const", r, 0.0))
                    else:
                        program.append(("assign", r, x))
                else:
                    # reductions end the stage: collected here, emitted after every elementwise op
                    reductions_at_end.append(("reduce", name, x, slot(_td(op))))
                    red_slots.append(op)
                    continue
            elif name in og_unary_names:
                x = operand_reg(op.args[0])
                r = new_reg()
                program.append((name, r, x))
            else:
                x, y = operand_reg(op.args[0]), operand_reg(op.args[1])
                r = new_reg()
                program.append((name, r, x, y))
            value_reg[op] = r
            if op in self.store_ops:
                program.append(("store", slot(_td(op)), r))

        program.extend(reductions_at_end)
        return operands, program, it_axes, red_axes, onehot_axes, take_axes, take_strides

    def _lower(self):
        operands, program, it_axes, red_axes, onehot_axes, take_axes, take_strides = self._collect()

        # ---- pass 2: dims = iteration axes with every operand's stride -----------------------
        def strides_over(td, axes):
            out = []
            for axis in axes:
                out.append(td.full_strides[td.axes.index(axis)] if axis in td.axes else 0)
            return out

        has_reduce = any(p[0] == "reduce" for p in program)
        if has_reduce:
            order = list(red_axes) + [a for a in it_axes if a not in red_axes]
        else:
            order = list(it_axes)
        dims = []
        for axis in order:
            tag = None
            if has_reduce and axis in red_axes:
                tag = "red"
            named = axis.name if (axis in onehot_axes or axis in take_axes) else None
            strides = [take_strides.get((s, axis), strides_over(td, [axis])[0]) for s, td in enumerate(operands)]
            dims.append(_Dim(axis.length, strides, tag, named))

        dims = self._coalesce(dims, has_reduce)
        outer, inner = self._split_outer(dims, has_reduce)

        # ---- pass 3: one spec per outer index -------------------------------------------------
        self.specs = []
        self.flex_bindings = []
        outer_shape = [d.length for d in outer]
        n_outer = int(np.prod(outer_shape, dtype=np.int64)) if outer else 1
        if any(d.length == 0 for d in dims):
            return
        for flat in range(n_outer):
            idx, rem = [], flat
            for n in reversed(outer_shape):
                idx.insert(0, rem % n)
                rem //= n
            offsets = [sum(i * d.strides[s] for i, d in zip(idx, outer)) for s in range(len(operands))]
            self.specs.append(self._build_spec(operands, program, inner, offsets, has_reduce))

    @staticmethod
    def _coalesce(dims, has_reduce):
        """Drop length-1 dims and merge neighbours every operand walks contiguously."""
        dims = [d for d in dims if d.length != 1 or d.named is not None]

        def mergeable(a, b):
            if a.tag != b.tag or a.named is not None or b.named is not None:
                return False
            return all(sa == sb * b.length for sa, sb in zip(a.strides, b.strides))

        if not has_reduce:
            # order by the strides of the operands (outermost first) so mergeable dims meet
            dims.sort(key=lambda d: tuple(-s for s in d.strides))
        else:
            red = [d for d in dims if d.tag == "red"]
            rest = [d for d in dims if d.tag != "red"]
            red.sort(key=lambda d: tuple(-s for s in d.strides))
            rest.sort(key=lambda d: tuple(-s for s in d.strides))
            dims = red + rest
        out = []
        for d in dims:
            if out and mergeable(out[-1], d):
                prev = out[-1]
                out[-1] = _Dim(prev.length * d.length, d.strides, prev.tag)   # neither is named
            else:
                out.append(d)
        return out

    @staticmethod
    def _split_outer(dims, has_reduce):
        """At most 3 dims go to the kernel (one reduced dim first); the rest loop on the host."""
        if has_reduce:
            red = [d for d in dims if d.tag == "red"]
            rest = [d for d in dims if d.tag != "red"]
            if len(red) == 0:
                red = [_Dim(1, [0] * len(dims[0].strides) if dims else [], "red")]
            if len(red) > 1:
                raise og_unsupported("reduction axes are not mergeable into one strided axis; "
                                     "make the operand contiguous in (reduced..., kept...) order")
            keep = rest[-2:] if len(rest) > 2 else rest
            outer = rest[:-2] if len(rest) > 2 else []
            return outer, red + keep
        keep = dims[-3:] if len(dims) > 3 else dims
        outer = dims[:-3] if len(dims) > 3 else []
        return outer, keep

    def _build_spec(self, operands, program, inner, offsets, has_reduce):
        t = self.transformer
        shape = [d.length for d in inner] or [1]
        nd = len(inner)
        sb = FusedSpecBuilder(shape)
        # Registers are fp32 (as in the reference's kernels wherever an integer meets a float:
        # float_ew2.py:615-641), which is exact for integers up to 2**24 only.  A kernel that
        # merely moves 32-bit integers declares them fp32: loads, register moves and stores pass
        # the bits through untouched, so the move is exact over the whole range.
        def is_dtype(td, numpy_type):
            return isinstance(td.dtype, (np.dtype, type)) and np.dtype(td.dtype) == np.dtype(numpy_type)

        moves_bits = (all(p[0] in ("load", "store", "assign") for p in program) and
                      any(all(is_dtype(td, kind) for td in operands) for kind in (np.int32, np.uint32)))
        for s, td in enumerate(operands):
            view = t.get_tensor_description_tensor_view(td)
            strides = [d.strides[s] for d in inner] or [0]
            dtype = t.ngh_dtype(np.dtype(np.float32) if moves_bits else td.dtype)
            slot = sb.tensor(view.ptr + offsets[s] * view.itemsize, strides, dtype,
                             take_extent=self.take_extents.get(s, 0))
            assert slot == s
        read, written = _emit_program(sb, program, inner)
        spec = sb.build()
        index = len(self.specs)
        spec.rng_seed = (t.rng_seed * 0x9E3779B1 + index * 0x85EBCA77 + self.kernel_number) & 0xFFFFFFFF
        for s, td in enumerate(operands):
            entry = t.flex_entry_of(td)
            if entry is not None:
                self.flex_bindings.append((index, s, entry, s in written))
        self.spec_uses.append([(td.base, s in read, s in written) for s, td in enumerate(operands)])
        t.runtime.validate_fused(spec)
        return spec

    def buffer_uses(self):
        """(base tensor description, is read, is written) of every operand."""
        return [u for uses in self.spec_uses for u in uses]

    def set_cache_hints(self, hint_of):
        for spec, uses in zip(self.specs, self.spec_uses):
            for s, (base, is_read, is_written) in enumerate(uses):
                spec.tensors[s].cache_hint = hint_of(base, is_read, is_written)

    def execute(self):
        rt = self.transformer.runtime
        for spec in self.specs:
            rt.launch_fused(spec)
            if self.n_rng_streams:
                spec.rng_counter = (spec.rng_counter + 1) & 0xFFFFFFFF    # fresh numbers next time

    def describe(self):
        rt = self.transformer.runtime
        return [[rt.describe_fused(spec, s) for s in range(spec.n_stages)] for spec in self.specs]


og_unary_names = set(_UNARY_NAMES.values())


def og_unsupported(msg):
    return NotImplementedError("hipgpu: " + msg)


class CopyKernel(HipKernel):
    """ContiguousOp: strided device copy (tensor_ops.py:137-204 DimShuffleKernel)."""

    def __init__(self, transformer, op):
        super(CopyKernel, self).__init__(transformer)
        self.op = op

    def bind_buffers(self):
        t = self.transformer
        src_td = _td(self.op.args[0].forwarded)
        dst_td = _td(self.op)
        self.src = t.get_tensor_description_tensor_view(src_td)
        self.dst = t.get_tensor_description_tensor_view(dst_td)
        self.shape = dst_td.shape
        order = [src_td.axes.index(a) for a in dst_td.axes]
        self.src_strides = [src_td.full_strides[i] for i in order]
        self.dst_strides = list(dst_td.full_strides)
        super(CopyKernel, self).bind_buffers()

    def buffer_uses(self):
        return [(_td(self.op.args[0].forwarded).base, True, False),
                (_td(self.op).base, False, True)]

    def describe(self):
        return [["copy_strided"]]

    def execute(self):
        self.transformer.runtime.copy_strided(self.dst.ptr, self.src.ptr, self.shape,
                                              self.dst_strides, self.src_strides, self.dst.itemsize)


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


class _ChainScratch(object):
    """An operand of a chain that is no tensor of the graph: one row of a statistics tensor, taken
    over for an intermediate (what a tensor description tells the merge, and its address)."""

    def __init__(self, base, ptr, axes, row):
        self.base, self.ptr, self.axes, self.offset = base, ptr, og.make_axes(axes), ("row", row)
        self.dtype = np.dtype(np.float32)
        strides, step = [], 1
        for a in reversed(list(axes)):
            strides.insert(0, step)
            step *= a.length
        self.full_strides = tuple(strides)


class ChainKernel(HipKernel):
    """Consecutive fused kernels over the same rows, merged: the STAGES of one spec.

    Reductions along the rows whose results the next kernels read back, elementwise passes over
    the same rows -- the maximum, the sum of exponentials and the normalised result of a softmax
    -- which the library runs in one kernel when it can (ngh_plan_chain; the reference's
    compound kernels run their stages inside one launch the same way, float_ew2.py:1135-1483).
    The operand then crosses the memory interface once instead of once per kernel.

    Chains are compiled programs: while the library has none for this spec (none built in, the
    run-time compiler not done yet, or switched off) the members run one by one as they would
    have alone, with the programs they match by themselves.
    """

    def __init__(self, transformer, members, spec, uses):
        super(ChainKernel, self).__init__(transformer)
        self.members = list(members)
        self.name = self.members[0].name
        self.ops = [op for m in self.members for op in getattr(m, "ops", None) or [m.op]]
        self.specs = [spec]
        self.spec_uses = [uses]
        for m in self.members:
            m.bind_buffers()
        self.buffers_bound = True
        self.ready = False
        self.programs_changed()

    def programs_changed(self):
        """Called when compiled programs may have been added to the library's table."""
        if not self.ready:
            self.ready = hiplib.plan_chain(self.specs[0])["special"] >= 0

    @classmethod
    def merged(cls, transformer, members):
        """The ChainKernel of `members`, or None when they do not form a row chain."""
        if isinstance(members[0], MomentsKernel):
            parts = cls._parts_after_moments(transformer, members[0], members[1:])
        elif any(isinstance(m, MomentsKernel) for m in members):
            parts = None
        else:
            parts = [m._collect() for m in members]
        return None if parts is None else cls._merge_parts(transformer, members, parts)

    @staticmethod
    def _parts_after_moments(t, moments, rest):
        """Mean, variance and 1/sqrt(variance + eps) of rows, and the kernels that use them, as
        stages: sum(x); sum((x - sum / n)^2); then the kernels, each load of a statistic replaced
        by its value computed from the two sums -- the statements ng.mean and ng.variance stand
        for (op_graph.py:4007-4009, 4252-4266).  When nothing outside `rest` reads the statistics
        the two sums go where those would have gone; else the sums get memory of their own and
        a stage in between writes the statistics out, one value per row."""
        if not rest or any(type(k) is not FusedKernel for k in rest):
            return None
        op = moments.op
        mom_base = _td(op).base
        readers, returned = t._usage_maps()
        inside = set(o for k in rest for o in k.ops)
        private = mom_base not in returned and all(u in inside for u in readers.get(mom_base, ()))
        moments.bind_buffers()
        x_td = _td(op.args[0].forwarded)
        n = float(op.reduction_axes.size)
        kept = [a for a in x_td.axes if a not in op.reduction_axes]
        rows = moments.rows
        stats = [_ChainScratch(mom_base, moments.out.ptr + i * rows * 4, kept, i) for i in range(3)]
        if private:
            sums = stats[:2]
        else:
            if getattr(moments, "chain_scratch", None) is None:
                moments.chain_scratch = t.runtime.malloc(2 * rows * 4)       # (freed with the runtime)
            own = object()
            sums = [_ChainScratch(own, moments.chain_scratch + i * rows * 4, kept, i) for i in range(2)]
        parts = [([x_td, sums[0]], [("load", 0, 0), ("reduce", "sum", 0, 1)],
                  x_td.axes, op.reduction_axes, [], [], {})]
        need_var = False
        later = []
        for k in rest:
            operands, program, it_axes, r_axes, onehot_axes, take_axes, take_strides = k._collect()
            row_of = {}
            for s, td in enumerate(operands):
                if td.base is mom_base:
                    view = t.get_tensor_description_tensor_view(td)
                    row_of[s] = (view.ptr - moments.out.ptr) // (rows * 4)
                    if row_of[s] not in (0, 1, 2) or (view.ptr - moments.out.ptr) % (rows * 4):
                        return None
            if any(ins[0] in ("store", "reduce") and ins[1 if ins[0] == "store" else 3] in row_of for ins in program):
                return None
            new_operands = [td for s, td in enumerate(operands) if s not in row_of]
            slot_map = {s: i for i, s in enumerate(s for s in range(len(operands)) if s not in row_of)}
            s0, s1 = len(new_operands), len(new_operands) + 1
            new_operands += sums
            next_reg = [1 + max([ins[1] for ins in program if ins[0] not in ("store", "store_trunc", "reduce")] + [0])]

            def reg():
                next_reg[0] += 1
                return next_reg[0] - 1
            new_program = []
            for ins in program:
                if ins[0] == "load" and ins[2] in row_of:
                    row = row_of[ins[2]]
                    total, count = reg(), reg()
                    new_program += [("load", total, s0 if row == 0 else s1), ("const", count, n)]
                    if row < 2:
                        new_program.append(("div", ins[1], total, count))
                    else:
                        var, eps, shifted, root = reg(), reg(), reg(), reg()
                        new_program += [("div", var, total, count), ("const", eps, float(op.epsilon)),
                                        ("add", shifted, var, eps), ("sqrt", root, shifted), ("rcp", ins[1], root)]
                    need_var = need_var or row > 0
                elif ins[0] == "load":
                    new_program.append((ins[0], ins[1], slot_map[ins[2]]))
                elif ins[0] == "store":
                    new_program.append((ins[0], slot_map[ins[1]], ins[2]))
                elif ins[0] == "reduce":
                    new_program.append((ins[0], ins[1], ins[2], slot_map[ins[3]]))
                else:
                    new_program.append(ins)
            later.append((new_operands, new_program, it_axes, r_axes, onehot_axes, take_axes, take_strides))
        if need_var or not private:
            parts.append(([x_td, sums[0], sums[1]],
                          [("load", 0, 0), ("load", 1, 1), ("const", 2, n), ("div", 3, 1, 2), ("sub", 4, 0, 3),
                           ("mul", 5, 4, 4), ("reduce", "sum", 5, 2)],
                          x_td.axes, op.reduction_axes, [], [], {}))
        if not private:
            # the statistics themselves, for their other readers
            program = [("load", 0, 0), ("load", 1, 1), ("const", 2, n), ("div", 3, 0, 2), ("store", 2, 3),
                       ("div", 4, 1, 2), ("store", 3, 4)]
            operands = [sums[0], sums[1], stats[0], stats[1]]
            if op.epsilon is not None:
                program += [("const", 5, float(op.epsilon)), ("add", 6, 4, 5), ("sqrt", 7, 6), ("rcp", 8, 7),
                            ("store", 4, 8)]
                operands.append(stats[2])
            parts.append((operands, program, x_td.axes, og.make_axes(()), [], [], {}))
        return parts + later

    @classmethod
    def _merge_parts(cls, t, members, parts):
        red_axes, all_axes = None, None
        for operands, program, it_axes, r_axes, onehot_axes, take_axes, _ in parts:
            if onehot_axes or take_axes or any(ins[0] in ("iota", "rng", "take", "store_trunc") for ins in program):
                return None
            # (axes compare by name: a window of an axis is another iteration space)
            extents = lambda axes: set((a.name, a.length) for a in axes)
            if all_axes is None:
                all_axes = it_axes
            elif extents(it_axes) != extents(all_axes):
                return None
            if any(ins[0] == "reduce" for ins in program):
                if red_axes is None:
                    red_axes = r_axes
                elif extents(r_axes) != extents(red_axes):
                    return None
            for td in operands:
                if not extents(td.axes) <= extents(all_axes):
                    return None
        if red_axes is None or not extents(red_axes) <= extents(all_axes):
            return None
        order = list(red_axes) + [a for a in all_axes if a not in red_axes]

        def walk(td):
            return [td.full_strides[td.axes.index(axis)] if axis in td.axes else 0 for axis in order]

        # one operand table for all stages; a view is known by the memory it walks over the chain's
        # axes (a reduction's result, and the same tensor broadcast along the row for the next
        # stage, are one operand)
        union, slot_of, programs = [], {}, []
        for operands, program, _, _, _, _, _ in parts:
            local = []
            for td in operands:
                key = (td.base, td.dtype, td.offset, tuple(walk(td)))
                if key not in slot_of:
                    slot_of[key] = len(union)
                    union.append(td)
                local.append(slot_of[key])
            remapped = []
            for ins in program:
                if ins[0] == "load":
                    ins = (ins[0], ins[1], local[ins[2]])
                elif ins[0] == "store":
                    ins = (ins[0], local[ins[1]], ins[2])
                elif ins[0] == "reduce":
                    ins = (ins[0], ins[1], ins[2], local[ins[3]])
                remapped.append(ins)
            programs.append(remapped)
        if len(union) > NGH_MAX_TENSORS:
            return None
        # what a stage writes, every stage must see through that one view
        written = set(ins[1] for prog in programs for ins in prog if ins[0] == "store")
        written |= set(ins[3] for prog in programs for ins in prog if ins[0] == "reduce")
        for s in written:
            for td in union:
                if td.base is union[s].base and td is not union[s] and \
                        not (isinstance(td, _ChainScratch) and isinstance(union[s], _ChainScratch)):
                    return None          # (two scratch operands are different rows of their tensor)
        walks = [walk(td) for td in union]
        dims = []
        for j, axis in enumerate(order):
            dims.append(_Dim(axis.length, [w[j] for w in walks], "red" if axis in red_axes else None))
        if any(d.length == 0 for d in dims):
            return None
        dims = FusedKernel._coalesce(dims, True)
        if len([d for d in dims if d.tag == "red"]) != 1 or len(dims) > 3:
            return None          # (the reduced axes do not walk as one, or axes are left to a host loop)
        _, inner = FusedKernel._split_outer(dims, True)
        sb = FusedSpecBuilder([d.length for d in inner] or [1])
        for s, td in enumerate(union):
            ptr = td.ptr if isinstance(td, _ChainScratch) else t.get_tensor_description_tensor_view(td).ptr
            sb.tensor(ptr, [d.strides[s] for d in inner] or [0], t.ngh_dtype(td.dtype))
        read, written = set(), set()
        try:
            for prog in programs:
                r, w = _emit_program(sb, prog, inner)
                read |= r
                written |= w
                sb.end_stage()
            spec = sb.build()
        except ValueError:           # more ops, constants or live values than one spec holds
            return None
        if not hiplib.plan_chain(spec)["eligible"]:
            return None
        t.runtime.validate_fused(spec)
        return cls(t, members, spec, [(td.base, s in read, s in written) for s, td in enumerate(union)])

    def buffer_uses(self):
        return list(self.spec_uses[0])

    def set_cache_hints(self, hint_of):
        whole = {}
        for s, (base, is_read, is_written) in enumerate(self.spec_uses[0]):
            self.specs[0].tensors[s].cache_hint = whole[base] = hint_of(base, is_read, is_written)
        # the members, for as long as they run by themselves: what one of them streams past the
        # cache another must not want to find there
        readers = {}
        for m in self.members:
            for base, is_read, _ in m.buffer_uses():
                if is_read:
                    readers[base] = readers.get(base, 0) + 1

        def member_hint(base, is_read, is_written):
            hint = whole.get(base, 0)
            if readers.get(base, 0) > 1:
                hint &= ~NGH_CACHE_STREAM_LOAD
            if readers.get(base, 0) > 0:
                hint &= ~NGH_CACHE_STREAM_STORE
            return hint
        for m in self.members:
            m.set_cache_hints(member_hint)

    def execute(self):
        if self.ready:
            self.transformer.runtime.launch_fused(self.specs[0])
        else:
            for m in self.members:
                m.execute()

    def describe(self):
        if not self.ready:
            return [d for m in self.members for d in m.describe()]
        rt = self.transformer.runtime
        return [[rt.describe_fused(spec, s) for s in range(spec.n_stages)] for spec in self.specs]


class KernelRun(HipKernel):
    """A run of consecutive fused kernels that may merge into ChainKernels.  Which do is decided
    when the buffers are bound (a spec needs addresses): greedily, the longest runs the library
    accepts as a row chain; a member that merges with no neighbour stays as it is.  The kernel
    group then takes the resulting kernels in this one's place (HipKernelGroup.bind)."""

    max_stages = 6               # NGH_MAX_STAGES

    def __init__(self, transformer, members):
        super(KernelRun, self).__init__(transformer)
        self.members = list(members)
        self.name = self.members[0].name
        self.kernels = []

    def bind_buffers(self):
        if not self.buffers_bound:
            self.kernels = []
            a, n = 0, len(self.members)
            while a < n:
                merged = None
                for b in range(min(n, a + self.max_stages), a + 1, -1):
                    merged = ChainKernel.merged(self.transformer, self.members[a:b])
                    if merged is not None:
                        break
                if merged is None:
                    self.members[a].bind_buffers()
                    self.kernels.append(self.members[a])
                    a += 1
                else:
                    self.kernels.append(merged)
                    a = b
        super(KernelRun, self).bind_buffers()

    @property
    def ops(self):
        return [op for m in self.members for op in getattr(m, "ops", None) or [m.op]]

    @property
    def specs(self):
        return [spec for k in self.kernels for spec in getattr(k, "specs", [])]

    def buffer_uses(self):
        return [u for k in self.kernels for u in k.buffer_uses()]

    def set_cache_hints(self, hint_of):
        for k in self.kernels:
            k.set_cache_hints(hint_of)

    def execute(self):
        for k in self.kernels:
            k.execute()

    def describe(self):
        return [d for k in self.kernels for d in k.describe()]


class HipKernelGroup(object):
    """The kernels of one computation and the loop that runs them (gputransform.py:348-522)."""

    def __init__(self, transformer, name):
        self.transformer = transformer
        self.name = name
        self.kernels = []
        self._bound = False

    def bind(self):
        """Lower every kernel, then tell each operand what the rest of the computation does
        with its buffer (the cache hints of the C ABI)."""
        for k in self.kernels:
            if not k.buffers_bound:
                k.bind_buffers()
        # (a run of kernels has settled which of them merge: its kernels take its place)
        self.kernels = [u for k in self.kernels for u in (k.kernels if isinstance(k, KernelRun) else [k])]
        self.assign_cache_hints()
        mode = self.transformer.jit
        if mode is True:
            # compile what would otherwise run on the interpreter (float_ew2.py:1553-1653: the
            # reference compiles every kernel of a computation at this point)
            from ngraph_hip.runtime import jit
            jit.ensure_programs(self.transformer.runtime, self.kernels, self.name,
                                min_elements=self.transformer.jit_min_elements)
            self.programs_changed()
        elif mode == "auto":
            # the same for the stages over large tensors, off the launch path: the computation
            # starts on the interpreter and picks the compiled kernels up when they are ready
            from ngraph_hip.runtime import jit
            self._programs = jit.start_background(self.transformer.runtime, self.kernels, self.name,
                                                  min_elements=self.transformer.jit_auto_min_elements,
                                                  small_min_elements=self.transformer.jit_min_elements)
        self._bound = True

    _programs = None

    def programs_changed(self):
        for k in self.kernels:
            if hasattr(k, "programs_changed"):
                k.programs_changed()

    def wait_for_programs(self, timeout=None):
        """Block until the kernels being compiled for this computation (jit="auto") are loaded;
        returns the compiler's message if it failed, else None."""
        if not self._bound:
            self.bind()
        if self._programs is None:
            return None
        self._programs.wait(timeout)
        error = self._programs.error
        self._programs = None
        self.programs_changed()
        return error

    def cancel_programs(self):
        if self._programs is not None:
            self._programs.cancel()
            self._programs = None

    def assign_cache_hints(self):
        uses = [k.buffer_uses() for k in self.kernels]
        readers = {}
        for i, ku in enumerate(uses):
            for base, is_read, _ in ku:
                if is_read:
                    readers.setdefault(base, set()).add(i)
        for i, k in enumerate(self.kernels):
            def hint_of(base, is_read, is_written, i=i):
                hint = 0
                r = readers.get(base, set())
                if is_read and r == {i}:
                    hint |= NGH_CACHE_STREAM_LOAD
                # a result that nothing here reads again; state updated in place is read by
                # the next execution and stays cacheable
                if is_written and not is_read and not any(j > i for j in r) \
                        and not getattr(base, "is_persistent", False):
                    hint |= NGH_CACHE_STREAM_STORE
                return hint
            k.set_cache_hints(hint_of)

    def setup_kernel_execute(self, kernel):
        pass

    def after_kernel_execute(self, kernel):
        pass

    def __call__(self):
        if not self._bound:
            self.bind()
        if self._programs is not None and self._programs.poll():
            self._programs = None
            self.programs_changed()
        for k in self.kernels:
            self.setup_kernel_execute(k)
            k.execute()
            self.after_kernel_execute(k)

    def profile(self, repeats=1, inner=1):
        """Per-kernel durations from HIP events on the launch stream.

        Each kernel is launched `inner` times back to back between one pair of events and the
        elapsed time divided by `inner` (amortises the event and launch overhead, so the
        figure is comparable with a profiler's kernel duration); this is repeated `repeats`
        times.  Returns [(kernel, [ms per launch])].  Kernels run out of their normal
        interleaving, so use it for per-kernel time, not for end-to-end time."""
        rt = self.transformer.runtime
        if not self._bound:
            self.bind()
        times = [[] for _ in self.kernels]
        for _ in range(repeats):
            for i, k in enumerate(self.kernels):
                self.setup_kernel_execute(k)
                rt.timer_begin()
                for _ in range(inner):
                    k.execute()
                times[i].append(rt.timer_end() / inner)
                self.after_kernel_execute(k)
        return list(zip(self.kernels, times))


# =============================================================================== fusion
class FusionPlanner(object):
    """Greedy grouping of consecutive fusable ops over one iteration space.

    A group is a run of elementwise ops, optionally ended by reductions that
    share their reduced axes (the stage rule of float_ew2.py:553-612).  An op
    starts a new group when its iteration axes differ, when it follows a
    reduction, when it would read or write memory the group touches through a
    different view, or when the kernel's operand / op / constant limits are hit.
    """

    small_tensor = 65536

    def __init__(self, transformer, fusion=True):
        self.transformer = transformer
        self.fusion = fusion

    def plan(self, ordered_ops, readers, returned):
        """List-schedule the ops: any dependency-respecting order is legal, so among the
        device ops that are ready prefer one the open group accepts.  Views, reads of state
        and sequencing ops cost nothing and are released as soon as they are ready."""
        ops = [op.forwarded for op in ordered_ops]
        position = {op: i for i, op in enumerate(ops)}
        pending, users = {}, {}
        for op in ops:
            deps = [d for d in op.all_deps if d in position]
            pending[op] = len(deps)
            for d in deps:
                users.setdefault(d, []).append(op)
        # device-op level dependencies, seen through views / reads / sequencing ops
        dev_deps, dev_users = {}, {}
        for op in ops:
            acc = set()
            for d in op.all_deps:
                if d not in position:
                    continue
                if d.is_device_op:
                    acc.add(d)
                else:
                    acc |= dev_deps.get(d, set())
            dev_deps[op] = acc
            if op.is_device_op:
                for d in acc:
                    dev_users.setdefault(d, set()).add(op)
        ready = [op for op in ops if pending[op] == 0]
        scheduled = set()
        groups, cur = [], None

        def release(op):
            scheduled.add(op)
            for u in users.get(op, ()):
                pending[u] -= 1
                if pending[u] == 0:
                    ready.append(u)

        def timely(op):
            """True unless every consumer of `op` still waits for something else: running such
            an op now would only park its result in memory until the consumer can run."""
            if isinstance(op, (og.ReductionOp, og.AssignOp, og.Fill)) or not op.is_tensor_op:
                return True
            if iteration_axes(op).size <= self.small_tensor:
                return True            # parking a small result costs nothing worth a split
            consumers = dev_users.get(op, ())
            if not consumers:
                return True
            for y in consumers:
                if all(d is op or d in scheduled or d in ready for d in dev_deps[y]):
                    return True
            return False

        def size(op):
            return iteration_axes(op).size if is_fusable(op) else 0

        while ready:
            free = [op for op in ready if not op.is_device_op]
            if free:
                for op in free:
                    ready.remove(op)
                    release(op)
                continue
            ready.sort(key=lambda op: position[op])
            pick = None
            if cur is not None and self.fusion:
                for op in ready:
                    if is_fusable(op) and timely(op) and cur.accepts(op, readers, returned):
                        pick = op
                        break
            if pick is None:
                # seed of the next group: a timely op if there is one, smallest space first
                # (scalars tend to be what the big kernels are waiting for)
                seeds = [op for op in ready if timely(op)] or ready
                pick = min(seeds, key=lambda op: (size(op), position[op])) if self.fusion else ready[0]
                if cur:
                    groups.append(cur)
                    cur = None
                if is_fusable(pick):
                    cur = _Group(pick, max_written_views=self.transformer.max_written_views)
                else:
                    groups.append(_Group(pick, fusable=False))
            else:
                cur.add(pick)
            ready.remove(pick)
            release(pick)
        if cur:
            groups.append(cur)
        if self.fusion:
            groups = self._recompute_across_groups(groups, readers, returned)
            groups = self._absorb_small_groups(groups, readers, returned)
            self._check_order(groups)
        for g in groups:
            if g.fusable:
                g.decide_stores(readers, returned)
        return groups

    @staticmethod
    def _check_order(groups):
        """Every value is produced before it is used: in an earlier kernel, or earlier in the same
        one.  (The passes that move ops between kernels must keep this; a violation is a planner
        bug, not a property of the user's graph.)"""
        seen = set()
        produced_somewhere = set(o for g in groups for o in g.ops)
        for g in groups:
            for o in g.ops:
                for a in o.args:
                    prod = _producer(a.forwarded)
                    if prod in produced_somewhere and prod not in seen and prod is not o and \
                            not isinstance(o, (og.AssignOp, og.Fill)):
                        raise RuntimeError("planner: {} is used by {} before any kernel computes it"
                                           .format(prod, o))
                seen.add(o)

    # -- recomputation instead of a round trip through memory -------------------------------------
    max_recompute_ops = 6

    def _recompute_across_groups(self, groups, readers, returned):
        """An elementwise result that later kernels need is normally written out and read back: two
        passes over a large tensor.  When the few ops that produce it can be repeated in those
        kernels from operands that are in memory anyway, at the price of at most one more large
        operand to read, repeating them is cheaper -- the rule of the reference's compound
        kernels, which re-emit the elementwise producers needed after a reduction
        (float_ew2.py:553-612), applied across kernels."""
        where = {}
        for gi, g in enumerate(groups):
            for op in g.ops:
                where[op] = gi
        plain = lambda op: (kernel_op_name(op) is not None and not isinstance(op, og.ReductionOp))
        for gi, g in enumerate(groups):
            if not g.fusable:
                continue
            for op in list(g.ops):
                if not plain(op) or iteration_axes(op).size <= self.small_tensor:
                    continue
                base = _td(op).base
                if base in returned:
                    continue
                inside = set(groups[gi].ops)
                outside = [u for u in readers.get(base, ()) if u not in inside]
                if not outside:
                    continue
                targets = sorted(set(where.get(u, -1) for u in outside))
                if targets[0] <= gi or not all(groups[hi].fusable for hi in targets):
                    continue
                chain = self._producer_chain(op, groups[gi], plain)
                if chain is None or len(chain) > self.max_recompute_ops:
                    continue
                leaves = self._outside_operands(chain)
                if self._written_between(leaves, groups, gi, targets[-1]):
                    continue
                rebuilt = {}
                for hi in targets:
                    h = groups[hi]
                    have = set(_view_key(td) for o in h.ops for td in h._operand_views(o)[0])
                    # (large next to the result itself: the per-row maxima of 131072 rows of 256
                    # elements are many, and still 1/256 of a pass; what counts is what the kernel
                    # would read on top of what it reads anyway: one more pass at most, a little over
                    # it with the maxima of ten-element columns)
                    size = iteration_axes(op).size
                    large = max(self.small_tensor, size // 16)
                    extra_large = [td for td in leaves
                                   if _view_key(td) not in have and _memory_elements(td) > large]
                    if len(extra_large) > 1 and sum(_memory_elements(td) for td in extra_large) > size + size // 4:
                        break
                    # the repeated ops are private to the kernel: whoever else needs them has them
                    new = _Group.rebuilt(h, chain, readers, returned, h.private)
                    if new is None:
                        break
                    rebuilt[hi] = new
                else:
                    for hi, new in rebuilt.items():
                        groups[hi] = new
                    groups[gi].never_store.add(op)
        return groups

    cheap_ops = ("add", "sub", "mul", "div", "neg", "abs", "sqrt", "rcp", "sqr", "minimum", "maximum", "assign")
    costly_ops = ("log", "exp", "safelog", "log2", "exp2")

    def _absorb_small_groups(self, groups, readers, returned):
        """A kernel over a few elements (per-channel factors between two passes over a big tensor)
        costs a launch, several microseconds, for nanoseconds of work.  When it consists of a few
        cheap elementwise ops and everything it produces is only read by later kernels whose axes
        include its own, those kernels repeat its ops themselves -- per element, from operands
        that are broadcast loads -- and the small kernel disappears."""
        holders = {}        # an op may have been repeated in several kernels by now
        for gi, g in enumerate(groups):
            for op in g.ops:
                holders.setdefault(op, set()).add(gi)
        gone = set()
        for gi, g in enumerate(groups):
            if not g.fusable or len(g.ops) > self.max_recompute_ops or \
                    g.axes.size > self.small_tensor or \
                    not all(kernel_op_name(o) in self.cheap_ops + self.costly_ops for o in g.ops):
                continue
            # (a logarithm or exponential per row: repeated by a kernel with at least 64 elements
            # a row, it is one such op per 4-element chunk at most, and none where the kernels
            # merge into a row chain, whose stages compute a row's values once)
            costly = any(kernel_op_name(o) in self.costly_ops for o in g.ops)
            inside = set(g.ops)
            targets, ok = set(), True
            for op in g.ops:
                base = _td(op).base
                if base in returned:
                    ok = False
                    break
                for u in readers.get(base, ()):
                    if u in inside:
                        continue
                    for hi in holders.get(u, (-1,)):
                        if hi <= gi or hi in gone or not groups[hi].fusable or \
                                not g.axes.is_sub_set(groups[hi].axes) or \
                                groups[hi].axes.size < 16 * g.axes.size or \
                                (costly and groups[hi].axes.size < 64 * g.axes.size):
                            ok = False
                            break
                        targets.add(hi)
                    if not ok:
                        break
                if not ok:
                    break
            if not ok or not targets:
                continue
            if self._written_between(self._outside_operands(g.ops), groups, gi, max(targets)):
                continue
            rebuilt = {}
            for hi in sorted(targets):
                h = groups[hi]
                new = _Group.rebuilt(h, g.ops, readers, returned, inside | h.private)
                if new is None:
                    break
                rebuilt[hi] = new
            else:
                for hi, new in rebuilt.items():
                    groups[hi] = new
                    for o in inside:
                        holders[o].add(hi)
                for o in inside:
                    holders[o].discard(gi)
                gone.add(gi)
        return [g for gi, g in enumerate(groups) if gi not in gone]

    @staticmethod
    def _producer_chain(op, group, plain):
        """The ops of `group`, in its order, that `op` is computed from inside the group; None if
        one of them is not a plain elementwise op."""
        index = {o: i for i, o in enumerate(group.ops)}
        need, stack = set(), [op]
        while stack:
            o = stack.pop()
            if o in need:
                continue
            if not plain(o):
                return None
            need.add(o)
            for a in o.args:
                prod = _producer(a.forwarded)
                if prod in index and index[prod] < index[o]:
                    stack.append(prod)
        return [o for o in group.ops if o in need]

    @staticmethod
    def _outside_operands(chain):
        inside = set(_td(o).base for o in chain)
        out = []
        for o in chain:
            for a in o.args:
                a = a.forwarded
                if _scalar_constant_value(a) is not None:
                    continue
                td = _td(a)
                if td.base not in inside:
                    out.append(td)
        return out

    @staticmethod
    def _written_between(leaves, groups, first, last):
        bases = set(td.base for td in leaves)
        for g in groups[first:last + 1]:
            for o in g.ops:
                if isinstance(o, (og.AssignOp, og.Fill)) and \
                        _td(o.args[0].forwarded).base in bases:
                    return True
        return False


class _Group(object):
    def __init__(self, op, fusable=True, max_written_views=NGH_MAX_TENSORS, axes=None, private=()):
        self.private = set(private)   # repeated ops: their results only ever live in registers
        self.ops = [op]
        self.fusable = fusable
        self.store_ops = set()
        self.never_store = set()      # results every outside reader recomputes for itself
        self.max_written_views = max_written_views    # flex kernels: one statistics slot per result
        self.n_written_views = 0
        if fusable:
            self.axes = iteration_axes(op) if axes is None else axes
            self.absorbed = set()     # ops over a subset of the axes, repeated along the others
            self.has_reduce = False
            self.red_axes = None
            self.read_views = {}     # base -> set(view keys)
            self.write_views = {}
            self.n_ops = 0
            self.n_consts = 0
            self.n_reds = 0
            self._account(op)

    def _operand_views(self, op):
        reads, writes = [], []
        if isinstance(op, og.AssignOp):
            writes.append(_td(op.args[0].forwarded))
            srcs = [op.args[1]]
        elif isinstance(op, og.Fill):
            writes.append(_td(op.args[0].forwarded))
            srcs = []
        else:
            writes.append(_td(op))
            srcs = list(op.args)
        for a in srcs:
            a = a.forwarded
            if _scalar_constant_value(a) is not None:
                continue
            reads.append(_td(a))
        return reads, writes

    def _account(self, op):
        reads, writes = self._operand_views(op)
        for td in reads:
            self.read_views.setdefault(td.base, set()).add(td.parameter_key)
        if op not in self.private:
            for td in writes:
                self.write_views.setdefault(td.base, set()).add(td.parameter_key)
        self.n_ops += 4
        self.n_consts += sum(1 for a in op.args if _scalar_constant_value(a.forwarded) is not None)
        if isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1:
            self.has_reduce = True
            self.red_axes = op.reduction_axes
            self.n_reds += 1

    def _memory_operands(self, candidate, readers, returned):
        """Operand slots the kernel would need with `candidate` added: buffers read from
        outside the group plus results something outside the group can see."""
        ops = self.ops + [candidate]
        inside = set(ops)
        produced = set()
        for op in ops:
            if op.is_tensor_op and not isinstance(op, (og.AssignOp, og.Fill)):
                produced.add(_td(op).base)
        views, written = set(), set()
        for op in ops:
            reads, writes = self._operand_views(op)
            for td in reads:
                if td.base not in produced:
                    views.add(_view_key(td))
            if isinstance(op, (og.AssignOp, og.Fill)):
                written.update(_view_key(td) for td in writes)
            else:
                base = _td(op).base
                if base in returned or isinstance(op, og.ReductionOp) or \
                        any(u not in inside for u in readers.get(base, ())):
                    written.add(_view_key(_td(op)))
        self.n_written_views = len(written)
        return len(views | written)

    def axes_fit(self, op, absorb=False):
        """Does op iterate over the group's axes -- or, for a cheap op of a smaller kernel that is
        repeated along the axes it lacks (`absorb`), over some of them?"""
        axes = iteration_axes(op)
        if not (axes.is_sub_set(self.axes) if absorb else axes.is_equal_set(self.axes)):
            return False
        return axes.lengths == tuple(self.axes[self.axes.index(a)].length for a in axes)

    @classmethod
    def rebuilt(cls, h, first, readers, returned, private):
        """The group `h` with the ops `first` (repeated from an earlier kernel, results private to
        this one) put in front; None if the rules of a group do not allow it."""
        # `first` is closed under its producers and reads only memory no kernel from its own to this
        # one writes, so those of its ops that h already repeats can move to the front with it
        ops = list(first) + [o for o in h.ops if o not in first]
        new = cls(ops[0], max_written_views=h.max_written_views, axes=h.axes, private=private)
        if not new.axes_fit(ops[0], ops[0] in new.private):
            return None
        for o in ops[1:]:
            if not new.accepts(o, readers, returned, absorb=o in new.private):
                return None
            new.add(o)
        new.never_store = set(h.never_store) | set(o for o in first if o not in h.ops)
        return new

    def accepts(self, op, readers, returned, absorb=False):
        if not self.axes_fit(op, absorb):
            return False
        is_red = isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1
        if self.has_reduce:
            if not is_red or not op.reduction_axes.is_equal_set(self.red_axes):
                return False
            if self.n_reds >= NGH_MAX_REDUCTIONS:
                return False
        reads, writes = self._operand_views(op)
        for td in reads:
            # reading what the group wrote is fine through the very same view only
            w = self.write_views.get(td.base)
            if w is not None and w != {td.parameter_key}:
                return False
        for td in writes:
            r = self.read_views.get(td.base)
            if r is not None and r != {td.parameter_key}:
                return False
            w = self.write_views.get(td.base)
            if w is not None and w != {td.parameter_key}:
                return False
        if is_red and not self._reduced_axes_mergeable(op, readers, returned):
            # the operands the fused kernel would read do not walk the reduced axes as one
            # strided axis: leave the reduction to a kernel of its own, whose argument is a
            # temporary in a layout that does (ReductionLayoutPass saw to that)
            return False
        if self._memory_operands(op, readers, returned) > NGH_MAX_TENSORS:
            return False
        if self.n_written_views > self.max_written_views:
            return False
        if self.n_ops + 4 > NGH_MAX_OPS or self.n_consts + 2 > NGH_MAX_CONSTS:
            return False
        if self._max_live(self.ops + [op]) + 4 > NGH_MAX_REGS:
            return False
        return True

    def _reduced_axes_mergeable(self, red_op, readers, returned):
        """Can every memory operand of the group plus `red_op` -- what it reads from outside and
        the elementwise results it has to write out -- walk red_op's reduced axes as ONE strided
        axis, in one common axis order?  (The kernels reduce over a single axis.)"""
        ops = self.ops + [red_op]
        inside = set(ops)
        produced = set(_td(op).base for op in ops
                       if op.is_tensor_op and not isinstance(op, (og.AssignOp, og.Fill)))
        tds = []
        for op in ops:
            reads, writes = self._operand_views(op)
            for td in reads:
                if td.base not in produced:
                    tds.append(td)
            if isinstance(op, (og.AssignOp, og.Fill)):
                tds.extend(writes)
            elif not (isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1):
                # (a reduction over axes of length 1 is an elementwise assignment)
                base = _td(op).base
                if base in returned or any(u not in inside for u in readers.get(base, ())):
                    tds.append(_td(op))
        red = [a for a in red_op.reduction_axes if a.length != 1]
        if len(red) < 2:
            return True

        def strides(td):
            return [td.full_strides[td.axes.index(a)] if a in td.axes else 0 for a in red]
        rows = [strides(td) for td in tds]
        rows = [r for r in rows if any(r)]
        if not rows:
            return True
        order = sorted(range(len(red)), key=lambda i: tuple(-r[i] for r in rows))
        for r in rows:
            for i, j in zip(order[:-1], order[1:]):
                if r[i] != r[j] * red[j].length:
                    return False
        return True

    @staticmethod
    def _max_live(ops):
        """Upper estimate of the registers the group's program keeps alive at once: a value
        (an op's result, or an operand loaded from memory at its first use) lives until its
        last use inside the group; constants are loaded where they are used."""
        index = {op: i for i, op in enumerate(ops)}
        born, last = {}, {}
        for i, op in enumerate(ops):
            srcs = op.args[1:] if isinstance(op, og.AssignOp) else (() if isinstance(op, og.Fill) else op.args)
            if isinstance(op, (og.RngOp,)):
                srcs = ()
            for a in srcs:
                a = a.forwarded
                if _scalar_constant_value(a) is not None:
                    continue
                prod = _producer(a)
                key = prod if prod in index and index[prod] < i else _view_key(_td(a))
                born.setdefault(key, index[prod] if key is prod else i)
                last[key] = i
            born.setdefault(op, i)
            last.setdefault(op, i)
        events = [0] * (len(ops) + 1)
        for key, b in born.items():
            events[b] += 1
            events[last[key]] -= 1          # dies at its last use: the result may take its register
        live = peak = 0
        for i in range(len(ops)):
            live += events[i]
            peak = max(peak, live + 3)      # + the op's transient constants and result
        return peak

    def add(self, op):
        self.ops.append(op)
        self._account(op)

    def decide_stores(self, readers, returned):
        """A result goes to memory only if something outside the group can see it."""
        inside = set(self.ops)
        for op in self.ops:
            if not op.is_tensor_op or isinstance(op, (og.AssignOp, og.Fill)):
                continue
            base = _td(op).base
            users = readers.get(base, ())
            if op in self.never_store:
                continue
            if base in returned or any(u not in inside for u in users):
                self.store_ops.add(op)
            elif isinstance(op, og.ReductionOp):
                self.store_ops.add(op)


# =============================================================================== transformer
class HipTransformer(ComputationGraphTransformer):
    """Transformer for executing graphs on an MI355X through libngraph_hip.so."""

    transformer_name = "hipgpu"
    default_rtol = 1e-05
    default_atol = 1e-08

    kernel_group_class = HipKernelGroup
    max_written_views = NGH_MAX_TENSORS      # results one fused kernel may write
    split_reductions = True                  # ReductionLayoutPass: reduce group by group of axes, no copy
    chain_kernels = True                     # consecutive kernels over the same rows run as stages of one spec

    def __init__(self, device_id=0, fusion=True, dry_run=False, fuse_moments=None, rng_seed=0, jit=None,
                 jit_min_elements=4096, jit_auto_min_elements=1 << 22, **kwargs):
        """dry_run=True lowers graphs to kernel specs without a device (no results can be
        read back); it exists so the host-side lowering can be inspected and tested.
        rng_seed keys the random fills (ng.uniform / ng.normal): same seed, same numbers.
        jit: how stages that the library has no compiled program for get one (the reference
        compiles every kernel of a computation when it is initialised, float_ew2.py:1553-1653).
        "auto" (the default unless NGH_JIT says otherwise): stages of at least
        jit_auto_min_elements elements are compiled in the background and swapped in when
        ready; True: every stage of at least jit_min_elements elements is compiled before the
        first launch; False: never."""
        from ngraph_hip.runtime import jit as _jit
        self.jit = _jit.normalize_mode(jit)
        self.jit_min_elements = int(jit_min_elements)
        self.jit_auto_min_elements = int(jit_auto_min_elements)
        try:
            self.runtime = DryRunRuntime() if dry_run else HipRuntime(device_id)
        except HipLibraryError as e:
            raise UnsupportedTransformerException("hipgpu needs libngraph_hip.so and an MI355X: %s" % e)
        super(HipTransformer, self).__init__(**kwargs)
        self.fusion = fusion
        self.rng_seed = int(rng_seed)
        self.n_kernels = 0
        self.kernel_groups = OrderedDict()
        self.graph_passes = [SimplePrune(), TensorSizeFold(), ConstantFoldPass(), SimplePrune()]
        if fusion if fuse_moments is None else fuse_moments:
            self.graph_passes.append(MomentsFusionPass())
        self.graph_passes.append(ReductionLayoutPass(split=self.split_reductions))

    # -- dtype mapping ---------------------------------------------------------------------
    def ngh_dtype(self, dtype):
        if not isinstance(dtype, np.dtype):
            return NGH_FLEX16
        # float_ew2.py:615-641 lists the storage types a compound kernel may touch
        for np_type, code in ((np.float32, NGH_F32), (np.int32, NGH_I32), (np.float16, NGH_F16),
                              (np.uint32, NGH_U32), (np.int16, NGH_I16), (np.int8, NGH_I8),
                              (np.uint8, NGH_U8)):
            if dtype == np_type:
                return code
        raise TypeError("hipgpu: unsupported tensor dtype %s" % dtype)

    def flex_entry_of(self, tensor_description):
        return None

    # -- hooks ---------------------------------------------------------------------------------
    def device_buffer_storage(self, bytes, dtype, name):
        return HipDeviceBufferStorage(self, bytes, dtype, name="a_" + name)

    def start_transform_allocate(self):
        pass

    def finish_transform_allocate(self):
        pass

    def gpu_kernel_group(self, name):
        return self.kernel_group_class(self, name)

    def _usage_maps(self):
        """Which device ops read each buffer, over every computation of this transformer."""
        readers, returned = {}, set()
        for op in self.ops:
            op = op.forwarded
            if op.is_device_op:
                srcs = op.args[1:] if isinstance(op, og.AssignOp) else \
                    (() if isinstance(op, og.Fill) else op.args)
                for a in srcs:
                    a = a.forwarded
                    if a.is_tensor_op:
                        readers.setdefault(_td(a).base, set()).add(op)
        for comp in self.computations:
            for v in comp.computation_op.values:
                v = v.forwarded
                if v.is_tensor_op:
                    returned.add(_td(v).base)
        return readers, returned

    def transform_ordered_ops(self, computation, ordered_ops, name):
        group = self.gpu_kernel_group(name)
        readers, returned = self._usage_maps()
        planner = FusionPlanner(self, fusion=self.fusion)
        for i, g in enumerate(planner.plan(ordered_ops, readers, returned)):
            if g.fusable:
                group.kernels.append(self.make_fused_kernel(g.ops, g.store_ops, "%s_k%d" % (name, i)))
            else:
                op = g.ops[0]
                if isinstance(op, og.ContiguousOp):
                    group.kernels.append(self.make_copy_kernel(op))
                elif isinstance(op, MomentsOp):
                    group.kernels.append(MomentsKernel(self, op))
                else:
                    raise ValueError("Unhandled op: {}".format(op))
        if self.chain_kernels and self.fusion:
            group.kernels = self._chained(group.kernels)
        self.kernel_groups[computation] = group
        computation.executor = group
        return name

    def _chained(self, kernels):
        """Runs of consecutive fused kernels with a reduction among them become KernelRuns."""
        out, run = [], []

        def flush():
            if len(run) >= 2 and (isinstance(run[0], MomentsKernel) or
                                  any(isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1
                                      for k in run for op in k.ops)):
                out.append(KernelRun(self, run))
            else:
                out.extend(run)
            del run[:]

        for k in kernels:
            if type(k) is FusedKernel:
                run.append(k)
            elif type(k) is MomentsKernel:
                # (the statistics of rows and the kernels that use them may merge as well)
                flush()
                run.append(k)
            else:
                flush()
                out.append(k)
        flush()
        return out

    def make_fused_kernel(self, ops, store_ops, name):
        return FusedKernel(self, ops, store_ops, name)

    def make_copy_kernel(self, op):
        return CopyKernel(self, op)

    def finish_transform(self):
        pass

    def allocate_storage(self):
        pass

    def close(self):
        for group in getattr(self, "kernel_groups", {}).values():
            if hasattr(group, "cancel_programs"):
                group.cancel_programs()
        rt = getattr(self, "runtime", None)
        if rt is not None:
            try:
                rt.sync()
            except Exception:
                pass
            rt.close()
            self.runtime = None
