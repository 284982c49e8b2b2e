"""Generate csrc/ngh_programs.inc: the op programs that get a pre-built kernel.

Each pattern below is built as an op graph, lowered by the same host code the
transformer uses (on a dry-run runtime, no GPU needed) and its streaming
elementwise stages are written out as compile-time program tables.  Because
the table comes from the lowering itself, a graph of the same structure lowers
to exactly these op sequences at run time and the library's structural match
finds the compiled kernel.  Run:  python csrc/gen_programs.py   (then rebuild).
tests/test_static_programs.py fails when the committed file is stale.
"""
from __future__ import print_function
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import numpy as np  # noqa: E402

import ngraph_hip as ng  # noqa: E402
import ngraph_hip.transformers as ngt  # noqa: E402
from ngraph_hip.frontends import neon  # noqa: E402
from ngraph_hip.runtime import hiplib  # noqa: E402

OUT = os.path.join(HERE, "ngh_programs.inc")


def _axes(**kw):
    return [ng.make_axis(length=v, name=k) for k, v in kw.items()]


def pattern_c1(t):
    H, W = _axes(H=1024, W=1024)
    x, a, b = ng.placeholder([H, W]), ng.placeholder(()), ng.placeholder(())
    return t.computation(ng.tanh(a * x + b) * ng.sigmoid(x), x, a, b)


def pattern_adam(t):
    P, = _axes(P=1 << 20)
    p, grad = ng.variable([P], initial_value=0.0), ng.placeholder([P])
    opt = neon.Adam()
    opt()
    updates, _, _ = opt.variable_update(p, grad)
    return t.computation(updates, grad)


def _rule_pattern(make):
    def build(t):
        P, = _axes(P=1 << 20)
        p, grad = ng.variable([P], initial_value=0.0), ng.placeholder([P])
        return t.computation(make().variable_update(p, grad)[0], grad)
    return build


def pattern_batchnorm(t):
    C, H, W, N = _axes(C=64, H=16, W=16, N=16)
    x = ng.placeholder([C, H, W, N])
    gamma, beta = ng.variable([C], initial_value=1.0), ng.variable([C], initial_value=0.0)
    y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    return t.computation([y, xmean, xvar], x)


def pattern_batchnorm_bprop(t):
    # backward of the same layer from an upstream error: two reductions in one pass (dbeta,
    # dgamma) and one elementwise pass (dx)
    C, H, W, N = _axes(C=64, H=16, W=16, N=16)
    x, err = ng.placeholder([C, H, W, N]), ng.placeholder([C, H, W, N])
    gamma, beta = ng.variable([C], initial_value=1.0), ng.variable([C], initial_value=0.0)
    y, _, _ = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    return t.computation([ng.deriv(y, x, error=err), ng.deriv(y, gamma, error=err),
                          ng.deriv(y, beta, error=err)], x, err)


def pattern_flex_relu(t):
    P, = _axes(P=1 << 20)
    x, w, b = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
    return t.computation(neon.rectlin(x * w + b), x, w, b)


def _reduction_pattern(fn, out_axis):
    def build(t):
        A, B = _axes(A=4096, B=4096)
        x = ng.placeholder([A, B])
        return t.computation(fn(x, out_axes=[A if out_axis == 0 else B]), x)
    return build


def _reduction_of(expr, out_axis, n_in=1):
    def build(t):
        A, B = _axes(A=4096, B=4096)
        xs = [ng.placeholder([A, B]) for _ in range(n_in)]
        return t.computation(expr(*xs, out_axes=[A if out_axis == 0 else B]), *xs)
    return build


def pattern_lstm_cell(t, Hn=1024, Nn=64):
    # LSTM cell on transposed storage (frontends/neon/layer.py:1630-1647): inputs contiguous
    # along H, results along N -- the tiled skeleton
    H, N, G = _axes(H=Hn, N=Nn, G=4 * Hn)
    gates_st, cprev_st = ng.placeholder([N, G]), ng.placeholder([N, H])
    gates = ng.axes_with_order(gates_st, [G, N])
    c_prev = ng.axes_with_order(cprev_st, [H, N])
    parts = {k: ng.cast_axes(ng.tensor_slice(gates, [slice(j * Hn, (j + 1) * Hn), slice(None)]), [H, N])
             for j, k in enumerate(("i", "f", "o", "g"))}
    h, c = neon.lstm_cell(parts, c_prev, H, None)
    return t.computation([c, h], gates_st, cprev_st)


def pattern_lstm_bias_gradient(t):
    # db = sum over N of gates [4H, N] stored transposed (frontends/neon/layer.py:1630-1647)
    N, G = _axes(N=64, G=4096)
    gates_st = ng.placeholder([N, G])
    gates = ng.axes_with_order(gates_st, [G, N])
    return t.computation(ng.sum(gates, out_axes=[G]), gates_st)


PATTERNS = [
    ("c1_tanh_sigmoid", "hipgpu", pattern_c1),
    ("adam", "hipgpu", pattern_adam),
    ("sgd_momentum", "hipgpu", _rule_pattern(lambda: neon.GradientDescentMomentum(0.1, 0.9))),
    ("sgd_momentum_wdecay", "hipgpu", _rule_pattern(lambda: neon.GradientDescentMomentum(0.1, 0.9, wdecay=0.01))),
    ("sgd_nesterov", "hipgpu", _rule_pattern(lambda: neon.GradientDescentMomentum(0.1, 0.9, nesterov=True))),
    ("rmsprop", "hipgpu", _rule_pattern(lambda: neon.RMSProp())),
    ("rmsprop_momentum_wdecay", "hipgpu", _rule_pattern(lambda: neon.RMSProp(wdecay=0.01, momentum_coef=0.5))),
    ("adagrad", "hipgpu", _rule_pattern(lambda: neon.Adagrad())),
    ("flex_adam", "flexhip", pattern_adam),
    ("flex_sgd_momentum", "flexhip", _rule_pattern(lambda: neon.GradientDescentMomentum(0.1, 0.9))),
    ("flex_rmsprop", "flexhip", _rule_pattern(lambda: neon.RMSProp())),
    ("batchnorm", "hipgpu", pattern_batchnorm),
    ("batchnorm_bprop", "hipgpu", pattern_batchnorm_bprop),
    ("flex_relu_fma", "flexhip", pattern_flex_relu),
    ("sum_along", "hipgpu", _reduction_pattern(ng.sum, 0)),
    ("sum_across", "hipgpu", _reduction_pattern(ng.sum, 1)),
    ("max_along", "hipgpu", _reduction_pattern(ng.max, 0)),
    ("max_across", "hipgpu", _reduction_pattern(ng.max, 1)),
    ("argmax_along", "hipgpu", _reduction_pattern(ng.argmax, 0)),
    ("argmax_across", "hipgpu", _reduction_pattern(ng.argmax, 1)),
    ("sum_of_squares_along", "hipgpu", _reduction_of(lambda x, out_axes: ng.sum(x * x, out_axes=out_axes), 0)),
    ("sum_of_squares_across", "hipgpu", _reduction_of(lambda x, out_axes: ng.sum(x * x, out_axes=out_axes), 1)),
    ("dot_along", "hipgpu", _reduction_of(lambda x, y, out_axes: ng.sum(x * y, out_axes=out_axes), 0, 2)),
    ("dot_across", "hipgpu", _reduction_of(lambda x, y, out_axes: ng.sum(x * y, out_axes=out_axes), 1, 2)),
    ("sum_across_small", "hipgpu", pattern_lstm_bias_gradient),
    ("lstm_cell", "hipgpu", pattern_lstm_cell),
    # the planner orders ops of large tensors differently (nothing above 65536 elements is
    # materialised early), which gives the cell a second program
    ("lstm_cell_large", "hipgpu", lambda t: pattern_lstm_cell(t, 2048, 512)),
]


def collect():
    """[(name, ops, dtypes, bcast, stat_slot, n_regs)] for every streaming stage of every pattern."""
    programs, seen = [], set()
    for name, backend, build in PATTERNS:
        if backend not in ngt.transformer_choices():
            continue
        t = ngt.make_transformer_factory(backend, dry_run=True)()
        f = build(t)
        t.initialize()
        k_index = 0
        for kernel in t.kernel_groups[f].kernels:
            kernel.bind_buffers()
            for spec in getattr(kernel, "specs", [])[:1]:
                for stage in range(spec.n_stages):
                    plan = hiplib.plan_fused(spec, stage)
                    st = spec.stages[stage]
                    family = plan["family"]
                    total = spec.shape[0] * spec.shape[1] * spec.shape[2]
                    # A one-element stage (a learning rule's step counter and rate factor) is worth a
                    # program of its own: the interpreter fetches the code of every op kind it meets
                    # with a cold instruction cache, several microseconds for twenty scalar ops.
                    scalar = total == 1 and family == 0 and not st.n_reductions
                    if family > 3 or (family == 0 and not scalar and (plan["V"] < 4 or st.n_reductions)):
                        continue
                    if family == 1 and spec.shape[0] // plan["V"] <= 64:
                        continue          # short rows run the several-rows-per-workgroup kernel
                    if total < 4096 and not scalar:
                        continue          # small stages are launch-bound; the interpreter is fine
                    if any(o.opcode >= hiplib.OPCODES["take"] for o in spec.ops[st.op_begin:st.op_end]):
                        continue          # lookups only run in the interpreter
                    ops = [(o.opcode, o.dst, o.a, o.b) for o in spec.ops[st.op_begin:st.op_end]]
                    fast = plan["perm"][2]
                    red_out = [st.red_out[r] for r in range(st.n_reductions)]
                    dtypes = [spec.tensors[i].dtype for i in range(spec.n_tensors)]
                    bcast = [1 if spec.tensors[i].strides[fast] == 0 else 0 for i in range(spec.n_tensors)]
                    stored = set(o[1] for o in ops if o[0] == hiplib.OPCODES["store"])
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
                                     [1 if i in stored else 0 for i in range(spec.n_tensors)]))
            k_index += 1
        t.close()
    return programs


def render(programs):
    lines = ["// GENERATED by gen_programs.py from the host lowering -- do not edit.",
             "// One entry per streaming elementwise op program that gets a pre-built kernel."]
    for i, (name, ops, dtypes, bcast, stat_slot, n_slots, n_regs, V, family, red_out, staged, loaded,
            stored) in enumerate(programs):
        lines.append("struct SP%d {  // %s" % (i, name))
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
        lines.append("};")
    lines.append("static const StaticEntry kStaticTable[] = {")
    for i, p in enumerate(programs):
        if p[8] == 0:
            launch = "&launch_static<SP%d>, nullptr, SP%d::staged, nullptr" % (i, i)
        elif p[8] == 3:
            launch = "nullptr, nullptr, SP%d::staged, &launch_static_tiled<SP%d>" % (i, i)
        else:
            launch = "nullptr, &launch_static_red<SP%d>, SP%d::staged, nullptr" % (i, i)
        lines.append('    {"%s", SP%d::family, SP%d::V, SP%d::n_ops, SP%d::ops, SP%d::n_tensors, SP%d::dtypes, '
                     'SP%d::bcast, SP%d::n_red, SP%d::red_out, %s},' % (p[0], i, i, i, i, i, i, i, i, i, launch))
    if not programs:
        lines.append('    {"none", 0, 4, 0, nullptr, 0, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr},')
    lines.append("};")
    lines.append("static const int kStaticCount = %d;" % len(programs))
    return "\n".join(lines) + "\n"


if __name__ == "__main__":
    text = render(collect())
    if "--check" in sys.argv:
        sys.exit(0 if open(OUT).read() == text else 1)
    with open(OUT, "w") as fh:
        fh.write(text)
    print("wrote", OUT)
