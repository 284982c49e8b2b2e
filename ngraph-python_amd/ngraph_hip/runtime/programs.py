"""Compiled op programs: from lowered kernels to the C++ tables the kernels are instantiated on.

A stage of a lowered fused kernel that one of the streaming / reduction / tiled skeletons can run
is described by a record (op list, operand types, which operands are broadcast along the fast
axis, vector width, skeleton); `render` writes records as the `struct SPn` tables and the entry
table that `csrc/ngh_special.h` instantiates kernels on.  Two users: `csrc/gen_programs.py`
writes the table that is built into the library, `jit.py` writes tables for the programs of a
user's computation and compiles them at run time (the reference generates and compiles CUDA C per
computation, float_ew2.py:1135-1483, :1553-1653).
"""
from ngraph_hip.runtime import hiplib


def stage_programs(kernels, name, seen=None, min_elements=4096, vector_only=False):
    """Records for every stage of `kernels` (lowered, buffers bound) that can run as a compiled
    program; `seen` holds the structural keys already recorded; `vector_only` leaves out
    elementwise stages without vector access (other than one-element ones)."""
    programs = []
    seen = set() if seen is None else seen
    k_index = 0
    # (a run of kernels that has settled which of them merge stands for those kernels)
    kernels = [u for k in kernels for u in (k.kernels if hasattr(k, "members") and hasattr(k, "kernels") else [k])]
    for kernel in kernels:
        for spec in getattr(kernel, "specs", [])[:1]:
            if spec.n_stages > 1:
                chain = _chain_program(spec, "%s_k%d" % (name, k_index), seen, min_elements)
                if chain is not None:
                    if chain:
                        programs.append(chain)
                    continue          # (its stages get no programs of their own)
            for stage in range(spec.n_stages):
                plan = hiplib.plan_fused(spec, stage)
                st = spec.stages[stage]
                family = plan["family"]
                total = spec.shape[0] * spec.shape[1] * spec.shape[2]
                # A one-element stage (a learning rule's step counter and rate factor) is worth a
                # program of its own: the interpreter fetches the code of every op kind it meets
                # with a cold instruction cache, several microseconds for twenty scalar ops.
                scalar = total == 1 and family == 0 and not st.n_reductions
                # An elementwise stage without vector access (V == 1: strided or misaligned views)
                # runs one element per lane with the operands' own strides; as a built-in program
                # only the one-element case is worth a table entry (`vector_only`).
                if family > 3 or (family == 0 and (st.n_reductions or plan["V"] in (2, 3))):
                    continue
                if family == 0 and plan["V"] == 1 and not scalar and vector_only:
                    continue
                if family == 1 and spec.shape[0] // plan["V"] <= 64 and vector_only:
                    continue          # short rows (several per workgroup): no table entry of their own
                if total < min_elements and not scalar:
                    continue          # small stages are launch-bound; the interpreter is fine
                codes = set(o.opcode for o in spec.ops[st.op_begin:st.op_end])
                if hiplib.OPCODES["store_trunc"] in codes and (family == 3 or vector_only):
                    continue          # the truncating store of a flex fill: not through the tiles, no built-in entries
                if codes & {hiplib.OPCODES["take"], hiplib.OPCODES["rng_uniform"], hiplib.OPCODES["rng_normal"]} \
                        and (family == 3 or vector_only):
                    continue          # lookups, random fills: not through the tiles, no built-in entries
                ops = [(o.opcode, o.dst, o.a, o.b) for o in spec.ops[st.op_begin:st.op_end]]
                fast = plan["perm"][2]
                red_out = [st.red_out[r] for r in range(st.n_reductions)]
                dtypes = [spec.tensors[i].dtype for i in range(spec.n_tensors)]
                bcast = [1 if spec.tensors[i].strides[fast] == 0 else 0 for i in range(spec.n_tensors)]
                stored = set(o[1] for o in ops if o[0] in (hiplib.OPCODES["store"], hiplib.OPCODES["store_trunc"]))
                loaded = set(o[2] for o in ops if o[0] == hiplib.OPCODES["load"])
                staged, n_staged = [], 0
                for i in range(spec.n_tensors):
                    st_i = spec.tensors[i].strides
                    if family == 3 and i in (stored | loaded) and st_i[plan["perm"][1]] == 1 and \
                            st_i[fast] not in (0, 1):
                        staged.append(n_staged)
                        n_staged += 1
                    else:
                        staged.append(-1)
                stat_slot, n_slots = [], 0
                for i in range(spec.n_tensors):
                    if i in stored and dtypes[i] == hiplib.NGH_FLEX16 and n_slots < 4:
                        stat_slot.append(n_slots)
                        n_slots += 1
                    else:
                        stat_slot.append(-1)
                key = (tuple(ops), tuple(dtypes), tuple(bcast), plan["V"], family, tuple(red_out), tuple(staged))
                if key in seen:
                    continue
                seen.add(key)
                programs.append(("%s_k%d" % (name, k_index), ops, dtypes, bcast, stat_slot,
                                 n_slots, spec.n_regs, plan["V"], family, red_out, staged,
                                 [1 if i in loaded else 0 for i in range(spec.n_tensors)],
                                 [1 if i in stored else 0 for i in range(spec.n_tensors)],
                                 plan["special"]))
        k_index += 1
    return programs


def _chain_program(spec, name, seen, min_elements):
    """The record of a spec whose stages run as one chain kernel; None when the spec is no chain,
    () when the chain is recorded already or too small to be worth a kernel.

    Family 4, a row chain: the second field holds the records of the stages, which are programs
    over rows along spec axis 0, 4 elements per lane.  Family 5, a column chain: the reduced
    axis (spec axis 0) is the strided one, the stages are programs 4 columns (spec axis 2) wide;
    their `rowshared` marks the operands that are the same for every row."""
    plan = hiplib.plan_chain(spec)
    if not plan["eligible"]:
        return None
    # (a chain is worth a kernel sooner than a single stage is: it saves launches, not only time
    # on the interpreter)
    if spec.shape[0] * spec.shape[1] * spec.shape[2] < min_elements // 16:
        return ()
    columns = plan["kind"] == "column"
    dtypes = [spec.tensors[i].dtype for i in range(spec.n_tensors)]
    if columns:
        ca = 2 if spec.shape[2] > 1 else 1           # (the columns: the last axis that has an extent)
        bcast = [1 if spec.tensors[i].strides[ca] == 0 else 0 for i in range(spec.n_tensors)]
        rowshared = [1 if spec.tensors[i].strides[0] == 0 else 0 for i in range(spec.n_tensors)]
    else:
        bcast = [1 if spec.tensors[i].strides[0] == 0 else 0 for i in range(spec.n_tensors)]
        # (the same for every row: a layer norm's gain and bias)
        rowshared = [1 if spec.tensors[i].strides[1] == 0 and spec.tensors[i].strides[2] == 0 else 0
                     for i in range(spec.n_tensors)]
    # the statistics slots of a row chain's flex16 results are the chain's: one per flex16 tensor
    # that a stage stores or reduces into, in operand order, the same in every stage's tables
    # (plan_row_chain numbers the kernel's arguments the same way)
    written = set()
    for stage in range(spec.n_stages):
        st = spec.stages[stage]
        written |= set(o.dst for o in spec.ops[st.op_begin:st.op_end] if o.opcode == hiplib.OPCODES["store"])
        written |= set(st.red_out[r] for r in range(st.n_reductions))
    stat_slot, n_slots = [], 0
    for i in range(spec.n_tensors):
        if not columns and i in written and dtypes[i] == hiplib.NGH_FLEX16:
            stat_slot.append(n_slots)
            n_slots += 1
        else:
            stat_slot.append(-1)
    members = []
    for stage in range(spec.n_stages):
        st = spec.stages[stage]
        if st.op_end == st.op_begin:
            continue
        ops = [(o.opcode, o.dst, o.a, o.b) for o in spec.ops[st.op_begin:st.op_end]]
        red_out = [st.red_out[r] for r in range(st.n_reductions)]
        stored = set(o[1] for o in ops if o[0] == hiplib.OPCODES["store"])
        loaded = set(o[2] for o in ops if o[0] == hiplib.OPCODES["load"])
        members.append(("%s_s%d" % (name, stage), ops, dtypes, bcast, stat_slot, n_slots, spec.n_regs, 4,
                        ((2 if columns else 1) if red_out else 0), red_out, [-1] * spec.n_tensors,
                        [1 if i in loaded else 0 for i in range(spec.n_tensors)],
                        [1 if i in stored else 0 for i in range(spec.n_tensors)], -1, rowshared))
    key = ("column chain" if columns else "chain", tuple(rowshared)) + \
        tuple((tuple(m[1]), tuple(m[2]), tuple(m[3]), m[8], tuple(m[9])) for m in members)
    if key in seen:
        return ()
    seen.add(key)
    return (name, members, dtypes, bcast, [], 0, spec.n_regs, 4, 5 if columns else 4, [], [], [], [], plan["special"])


def _render_struct(lines, struct, record):
    name, ops, dtypes, bcast, stat_slot, n_slots, n_regs, V, family, red_out, staged, loaded, stored, _ = record[:14]
    rowshared = record[14] if len(record) > 14 else [0] * len(dtypes)
    lines.append("struct %s {  // %s" % (struct, name))
    lines.append("    static constexpr int V = %d, n_ops = %d, n_regs = %d, n_tensors = %d, "
                 "n_stat_slots = %d, family = %d, n_red = %d;"
                 % (V, len(ops), max(n_regs, 1), len(dtypes), n_slots, family, len(red_out)))
    lines.append("    static constexpr int red_out[%d] = {%s};"
                 % (max(len(red_out), 1), ", ".join(map(str, red_out or [0]))))
    lines.append("    static constexpr ngh_op ops[%d] = {%s};"
                 % (len(ops), ", ".join("{%d,%d,%d,%d}" % o for o in ops)))
    lines.append("    static constexpr int dtypes[%d] = {%s};" % (len(dtypes), ", ".join(map(str, dtypes))))
    lines.append("    static constexpr unsigned char bcast[%d] = {%s};" % (len(bcast), ", ".join(map(str, bcast))))
    lines.append("    static constexpr int stat_slot[%d] = {%s};" % (len(stat_slot), ", ".join(map(str, stat_slot))))
    lines.append("    static constexpr int n_staged = %d;" % sum(1 for x in staged if x >= 0))
    lines.append("    static constexpr signed char staged[%d] = {%s};" % (len(staged), ", ".join(map(str, staged))))
    lines.append("    static constexpr unsigned char loaded[%d] = {%s};" % (len(loaded), ", ".join(map(str, loaded))))
    lines.append("    static constexpr unsigned char stored[%d] = {%s};" % (len(stored), ", ".join(map(str, stored))))
    lines.append("    static constexpr unsigned char rowshared[%d] = {%s};" % (len(rowshared), ", ".join(map(str, rowshared))))
    lines.append("};")


_ENTRY = ('{{"{1}", {0}::family, {0}::V, {0}::n_ops, {0}::ops, {0}::n_tensors, {0}::dtypes, '
          '{0}::bcast, {0}::n_red, {0}::red_out, {2}}},')


def render(programs, header, prefix="SP", table="kStaticTable", count="kStaticCount", pairs=None):
    """C++ text: one `struct <prefix>n` per record, the entry table and its length; with `pairs`
    [(name of a tiled elementwise program, name of a column reduction)] also the table of programs
    that one launch runs side by side (kPairTable / kPairCount)."""
    lines = list(header)
    for i, p in enumerate(programs):
        if p[8] in (4, 5):
            # a chain: the structs of its stages and the array of their entries (no launchers)
            for j, member in enumerate(p[1]):
                _render_struct(lines, "%s%d_%d" % (prefix, i, j), member)
            lines.append("static const StaticEntry %s%d_stages[] = {" % (prefix, i))
            for j, member in enumerate(p[1]):
                lines.append("    " + _ENTRY.format("%s%d_%d" % (prefix, i, j), member[0],
                                                    "nullptr, nullptr, nullptr, nullptr, 0, nullptr, "
                                                    "%s%d_%d::rowshared" % (prefix, i, j)))
            lines.append("};")
        else:
            _render_struct(lines, prefix + str(i), p)
    lines.append("static const StaticEntry %s[] = {" % table)
    for i, p in enumerate(programs):
        if p[8] in (4, 5):
            stages = ", ".join("%s%d_%d" % (prefix, i, j) for j in range(len(p[1])))
            lines.append('    {"%s", %d, 4, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, '
                         '%d, %s%d_stages, nullptr, &%s<%s>},'
                         % (p[0], p[8], len(p[1]), prefix, i,
                            "launch_static_chain" if p[8] == 4 else "launch_static_col_chain", stages))
            continue
        if p[8] == 0:
            launch = "&launch_static<{0}>, nullptr, {0}::staged, nullptr".format(prefix + str(i))
        elif p[8] == 3:
            launch = "nullptr, nullptr, {0}::staged, &launch_static_tiled<{0}>".format(prefix + str(i))
        else:
            launch = "nullptr, &launch_static_red<{0}>, {0}::staged, nullptr".format(prefix + str(i))
        lines.append("    " + _ENTRY.format(prefix + str(i), p[0], launch))
    if not programs:
        lines.append('    {"none", 0, 4, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr},')
    lines.append("};")
    lines.append("static const int %s = %d;" % (count, len(programs)))
    if pairs is not None:
        index = {p[0]: i for i, p in enumerate(programs)}
        lines.append("static const PairEntry kPairTable[] = {")
        for first, second in pairs:
            a, b = programs[index[first]], programs[index[second]]
            assert a[8] == 3 and b[8] == 2 and a[5] == 0 and b[5] == 0, (first, second)
            lines.append('    {"%s", "%s", &launch_static_pair<%s%d, %s%d>},' % (first, second, prefix, index[first], prefix, index[second]))
        if not pairs:
            lines.append('    {nullptr, nullptr, nullptr},')
        lines.append("};")
        lines.append("static const int kPairCount = %d;" % len(pairs))
    return "\n".join(lines) + "\n"
