"""Consecutive kernels over the same rows or columns as the stages of ONE spec, which the
library runs in one launch when it has the chain's program (the reference's compound kernels
run their stages inside one launch too: float_ew2.py:1135-1483).
"""
from __future__ import division

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.runtime import hiplib
from ngraph_hip.runtime.hiplib import (FusedSpecBuilder, NGH_MAX_TENSORS, NGH_CACHE_STREAM_LOAD,
                                       NGH_CACHE_STREAM_STORE)
from ngraph_hip.transformers.hipdevice import _td
from ngraph_hip.transformers.hiplowering import FusedKernel, HipKernel, _Dim, _emit_program
from ngraph_hip.transformers.hipmoments import MomentsKernel


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

    def __init__(self, transformer, members, spec, uses, operands=()):
        super(ChainKernel, self).__init__(transformer)
        self.members = list(members)
        self.operands = list(operands)        # tensor descriptions (or scratch rows) of the spec's operand slots
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
        if parts is None or any(getattr(m, "raw_slots", None) for m in members):
            return None      # (tensors bound for integer registers: a chain binds every operand by its own type)
        return cls._merge_parts(transformer, members, parts)

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
        return cls(t, members, spec, [(td.base, s in read, s in written) for s, td in enumerate(union)], union)

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
                    merged = self.transformer.chain_kernel_class.merged(self.transformer, self.members[a:b])
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
