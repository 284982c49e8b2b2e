"""Which ops of a computation share a kernel.  The reference's generator supports compounds of
several ops and stages (float_ew2.py:553-612, 1135-1429) but its transformer hands it one op at
a time (gputransform.py:381-391); the planner here groups them.
"""
from __future__ import division

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.runtime.hiplib import (NGH_MAX_TENSORS, NGH_MAX_OPS, NGH_MAX_CONSTS, NGH_MAX_REGS,
                                       NGH_MAX_REDUCTIONS)
from ngraph_hip.transformers.hipdevice import _td
from ngraph_hip.transformers.hiplowering import (kernel_op_name, is_fusable, iteration_axes,
                                                 _scalar_constant_value, _producer, _memory_elements,
                                                 _view_key)


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
