"""From a group of graph ops to kernel specs (the part of gputransform.py:124-345 and
float_ew2.py:289-338, 553-612 that prepares a compound kernel): op class -> kernel op name, the
operands of a group as views over at most three merged axes, its program over numbered
registers, and the kernels that launch it (`FusedKernel`) or copy a strided view (`CopyKernel`).
"""
from __future__ import division
from collections import OrderedDict

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.runtime.hiplib import FusedSpecBuilder
from ngraph_hip.transformers.hipdevice import _td

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


class _MixedIntegerUse(Exception):
    """A kernel would move an integer tensor as bits and also write it through a conversion."""


def _int_kind_of(dtype):
    """"i" for int32, "u" for uint32, else None."""
    if not isinstance(dtype, (np.dtype, type)):
        return None
    dtype = np.dtype(dtype)
    return "i" if dtype == np.dtype(np.int32) else ("u" if dtype == np.dtype(np.uint32) else None)


# Integer forms of the ops whose NumPy integer loop and whose C operator agree and wrap the same
# way (cputransform.py:512-761 hands integer arrays to the ufuncs as they are; division and
# remainder are not among them: NumPy divides integers in floating point and takes the floored
# remainder, C truncates).
_COMPARISONS = ("eq", "ne", "lt", "le", "gt", "ge")
_INT_UNARY = {"neg": "ineg", "abs": "iabs"}
_INT_BINARY = {
    "i": {"add": "iadd", "sub": "isub", "mul": "imul", "minimum": "imin", "maximum": "imax",
          "eq": "ieq", "ne": "ine", "lt": "ilt", "le": "ile", "gt": "igt", "ge": "ige"},
    "u": {"add": "iadd", "sub": "isub", "mul": "imul", "minimum": "umin", "maximum": "umax",
          "eq": "ieq", "ne": "ine", "lt": "ult", "le": "ule", "gt": "ugt", "ge": "uge"},
}


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

    integer_registers = True     # (a flex kernel has none: every tensor of it is flex16)

    def _collect(self):
        """Pass 1 of the lowering: the operands (views) the group touches and its program over
        symbolic registers; returns (operands, program, it_axes, red_axes, onehot_axes,
        take_axes, take_strides).  Sets self.raw_slots."""
        try:
            return self._collect_once()
        except _MixedIntegerUse:
            # an integer tensor that this kernel both moves as bits and writes through a
            # conversion: one binding cannot serve both, so the kernel keeps floats throughout
            self.integer_registers = False
            return self._collect_once()

    def _collect_once(self):
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
        # Registers that hold 32-bit integers as integers ("i": int32, "u": uint32) rather than
        # as floats: what the reference declares `int` / `unsigned int` (float_ew2.py:615-641).
        # Values loaded from int32 / uint32 tensors start out that way; an op all of whose
        # operands do is integer arithmetic (NumPy's integer loops, C's integer operators),
        # anything else converts them to float first.
        int_kind = {}            # symbolic register -> "i" | "u"
        self.raw_slots = set()   # operand slots whose 32-bit integers move as plain bits

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
            kind = _int_kind_of(td.dtype)
            if kind is not None and self.integer_registers and self.transformer.flex_entry_of(td) is None:
                if slot(td) in converted_slots:
                    raise _MixedIntegerUse()
                int_kind[r] = kind
                self.raw_slots.add(slot(td))
            value_reg[key] = r
            return r

        def as_float(r):
            """The register itself, or a float copy of the integer it holds."""
            kind = int_kind.get(r)
            if kind is None:
                return r
            f = new_reg()
            program.append(("i2f" if kind == "i" else "u2f", f, r))
            return f

        def store(td, r):
            """STORE of register r into the operand td: integers into an integer tensor of the
            same kind go as they are, anything else through the store's own conversion."""
            s_ = slot(td)
            kind = int_kind.get(r)
            if kind is not None and kind == _int_kind_of(td.dtype) and s_ not in converted_slots:
                self.raw_slots.add(s_)
                program.append(("store", s_, r))
                return
            converting(s_)
            program.append(("store", s_, as_float(r)))

        def converting(s_):
            """Slot s_ is written through the library's own conversion (a float into an integer
            tensor, a fill, a reduction's result)."""
            if s_ in self.raw_slots:
                raise _MixedIntegerUse()
            converted_slots.add(s_)

        converted_slots = set()  # integer tensors written through a conversion
        red_slots = []
        reductions_at_end = []
        for op in ops:
            name = kernel_op_name(op)
            if isinstance(op, og.AssignOp):
                target, val = op.args[0].forwarded, op.args[1].forwarded
                r = operand_reg(val)
                td = _td(target)
                store(td, r)
                value_reg[_view_key(td)] = r
                continue
            if isinstance(op, og.Fill):
                td = _td(op.args[0].forwarded)
                r = new_reg()
                program.append(("const", r, float(op.scalar)))
                converting(slot(td))
                program.append((self.fill_store, slot(td), r))
                value_reg[_view_key(td)] = r
                continue
            if isinstance(op, og.OneHotOp):
                x = as_float(operand_reg(op.args[0]))
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
                x = as_float(operand_reg(idx))
                lut_td = _td(lut)
                table = slot(lut_td)
                out_axis = op.axes[op.lut_axis]
                take_axes.append(out_axis)
                take_strides[(table, out_axis)] = lut_td.full_strides[op.lut_axis]
                self.take_extents[table] = lut_td.shape[op.lut_axis]
                r = new_reg()
                program.append(("take", r, x, table, out_axis))
            elif isinstance(op, og.ReductionOp):
                x = as_float(operand_reg(op.args[0]))
                if len(op.reduction_axes) == 0 or op.reduction_axes.size == 1:
                    # nothing to reduce: assign (gputransform.py:117-119, float_ew2.py:582-586)
                    r = new_reg()
                    if name in ("argmax", "argmin"):
                        program.append(("const", r, 0.0))
                    else:
                        program.append(("assign", r, x))
                else:
                    # reductions end the stage: collected here, emitted after every elementwise op
                    converting(slot(_td(op)))
                    reductions_at_end.append(("reduce", name, x, slot(_td(op))))
                    red_slots.append(op)
                    continue
            elif name in og_unary_names:
                x = operand_reg(op.args[0])
                r = new_reg()
                kind = int_kind.get(x)
                if kind == "i" and name in _INT_UNARY:
                    program.append((_INT_UNARY[name], r, x))
                    int_kind[r] = kind
                else:
                    program.append((name, r, as_float(x)))
            else:
                x, y = operand_reg(op.args[0]), operand_reg(op.args[1])
                r = new_reg()
                kind = int_kind.get(x)
                if kind is not None and kind == int_kind.get(y) and name in _INT_BINARY[kind]:
                    program.append((_INT_BINARY[kind][name], r, x, y))
                    if name not in _COMPARISONS:          # (a comparison gives 1.0 / 0.0)
                        int_kind[r] = kind
                else:
                    program.append((name, r, as_float(x), as_float(y)))
            if r in int_kind and _int_kind_of(op.dtype) != int_kind[r]:
                # the op's own type is not that integer type: its value is converted, as an
                # assignment to a `float` register converts in C
                r = as_float(r)
            value_reg[op] = r
            if op in self.store_ops:
                store(_td(op), r)

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
        # Integer tensors whose elements the program handles as integers (self.raw_slots: loaded
        # into integer registers, stored from them) are bound as fp32: LOAD, register moves and
        # STORE then pass their 32 bits through untouched; conversions are ops of the program.
        for s, td in enumerate(operands):
            view = t.get_tensor_description_tensor_view(td)
            strides = [d.strides[s] for d in inner] or [0]
            dtype = t.ngh_dtype(np.dtype(np.float32) if s in self.raw_slots else td.dtype)
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
