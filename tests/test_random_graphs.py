"""Randomly built graphs (fixed seeds): the HIP transformer against the NumPy oracle
transformer on the same graph and inputs.  Exercises the fusion planner and the lowering on
shapes nobody wrote by hand: broadcasts over axis subsets, reordered and sliced views,
reductions over several axes feeding further elementwise ops, results shared by several
consumers."""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
import oracle.cpu_transformer  # noqa: F401

UNARY = [ng.tanh, ng.negative, ng.absolute, ng.square, ng.sigmoid, lambda x: ng.sqrt(ng.absolute(x) + 0.5),
         lambda x: ng.exp(x * 0.25), lambda x: ng.log(ng.absolute(x) + 1.0), ng.sign]
BINARY = [ng.add, ng.subtract, ng.multiply, ng.maximum, ng.minimum, lambda a, b: a / (ng.absolute(b) + 1.0),
          lambda a, b: ng.greater(a, b), lambda a, b: ng.less_equal(a, b)]
REDUCE = [ng.sum, ng.max, ng.min, ng.mean]


def build(seed):
    rs = np.random.RandomState(seed)
    n_axes = rs.randint(2, 5)
    lengths = [int(rs.choice([1, 2, 3, 5, 8, 16, 33])) for _ in range(n_axes)]
    all_axes = [ng.make_axis(n, name="ax%d_%d" % (seed, i)) for i, n in enumerate(lengths)]
    inputs, values = [], []
    for _ in range(rs.randint(2, 5)):
        k = rs.randint(1, n_axes + 1)
        idx = sorted(rs.choice(n_axes, size=k, replace=False))
        if rs.rand() < 0.4:
            idx = list(rs.permutation(idx))                       # stored in another axis order
        axes = [all_axes[i] for i in idx]
        inputs.append(ng.placeholder(axes))
        values.append(rs.uniform(-2, 2, [a.length for a in axes]).astype(np.float32))
    pool = list(inputs)
    for _ in range(rs.randint(4, 14)):
        kind = rs.rand()
        if kind < 0.35:
            x = pool[rs.randint(len(pool))]
            node = UNARY[rs.randint(len(UNARY))](x)
        elif kind < 0.8:
            a, b = pool[rs.randint(len(pool))], pool[rs.randint(len(pool))]
            node = BINARY[rs.randint(len(BINARY))](a, b)
        else:
            x = pool[rs.randint(len(pool))]
            if len(x.axes) == 0:
                continue
            k = rs.randint(1, len(x.axes) + 1)
            red = [x.axes[i] for i in sorted(rs.choice(len(x.axes), size=k, replace=False))]
            node = REDUCE[rs.randint(len(REDUCE))](x, reduction_axes=ng.make_axes(red))
        pool.append(node)
    results = [pool[-1]] + [pool[i] for i in rs.choice(np.arange(len(inputs), len(pool)), size=min(2, len(pool) - len(inputs)),
                                                       replace=False)]
    return results, inputs, values


def run(backend, results, inputs, values, **kwargs):
    t = ngt.make_transformer_factory(backend, **kwargs)()
    try:
        f = t.computation(results, *inputs)
        return [np.array(r) for r in f(*values)]
    finally:
        t.close()


@pytest.mark.parametrize("seed", range(200))
def test_oracle_transformer_agrees_with_itself_unfused(seed):
    """CPU-only sanity of the generator: every graph builds and evaluates on the oracle."""
    results, inputs, values = build(seed)
    out = run("cpu", results, inputs, values)
    assert all(np.isfinite(o).all() for o in out)


@pytest.mark.gpu
@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "unfused"])
@pytest.mark.parametrize("seed", range(200))
def test_random_graph_matches_oracle(seed, fusion):
    results, inputs, values = build(seed)
    want = run("cpu", results, inputs, values)
    got = run("hipgpu", results, inputs, values, fusion=fusion)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-5)


# ------------------------------------------------------------------ second generator: larger shapes, views
def build_views(seed):
    """Larger tensors (vector, tiled and multi-segment kernels get chosen), up to five axes (the
    host loops over what does not fit three), sliced and reordered views as operands, argmax /
    prod reductions with explicit out_axes orders."""
    rs = np.random.RandomState(seed)
    n_axes = rs.randint(2, 6)
    lengths = [int(rs.choice([1, 2, 3, 4, 8, 16, 32, 64, 100])) for _ in range(n_axes)]
    while np.prod(lengths) > 400000:
        lengths[int(np.argmax(lengths))] //= 2
    all_axes = [ng.make_axis(n, name="bx%d_%d" % (seed, i)) for i, n in enumerate(lengths)]
    inputs, values, pool = [], [], []
    for _ in range(rs.randint(2, 4)):
        k = rs.randint(max(1, n_axes - 2), n_axes + 1)
        idx = list(rs.permutation(n_axes)[:k]) if rs.rand() < 0.5 else sorted(rs.choice(n_axes, size=k, replace=False))
        axes = [all_axes[i] for i in idx]
        p = ng.placeholder(axes)
        inputs.append(p)
        values.append(rs.uniform(-2, 2, [a.length for a in axes]).astype(np.float32))
        view = p
        if rs.rand() < 0.5 and len(axes) > 1:
            view = ng.axes_with_order(view, [axes[i] for i in rs.permutation(len(axes))])
        pool.append(view)
    # a sliced operand: a window of the first input along its first axis, renamed so it can
    # only meet operands through its other axes
    first = inputs[0]
    if first.axes[0].length >= 4:
        lo = int(rs.randint(0, first.axes[0].length // 2))
        hi = int(rs.randint(lo + 1, first.axes[0].length + 1))
        sl = ng.tensor_slice(first, [slice(lo, hi)] + [slice(None)] * (len(first.axes) - 1))
        pool.append(ng.sum(sl, reduction_axes=ng.make_axes([sl.axes[0]])) if len(sl.axes) > 1 else ng.sum(sl))
    for _ in range(rs.randint(5, 12)):
        kind = rs.rand()
        if kind < 0.3:
            node = UNARY[rs.randint(len(UNARY))](pool[rs.randint(len(pool))])
        elif kind < 0.75:
            node = BINARY[rs.randint(len(BINARY))](pool[rs.randint(len(pool))], pool[rs.randint(len(pool))])
        else:
            x = pool[rs.randint(len(pool))]
            if len(x.axes) == 0:
                continue
            which = rs.rand()
            if which < 0.25:
                node = ng.argmax(x, reduction_axes=ng.make_axes([x.axes[rs.randint(len(x.axes))]]))
            elif which < 0.4:
                node = ng.prod(x * 0.5, reduction_axes=ng.make_axes([x.axes[rs.randint(len(x.axes))]]))
            else:
                k = rs.randint(1, len(x.axes) + 1)
                red = [x.axes[i] for i in sorted(rs.choice(len(x.axes), size=k, replace=False))]
                kept = [a for a in x.axes if a not in red]
                out_axes = [kept[i] for i in rs.permutation(len(kept))]
                node = REDUCE[rs.randint(len(REDUCE))](x, out_axes=ng.make_axes(out_axes))
        pool.append(node)
    n_in = len(inputs)
    picks = rs.choice(np.arange(n_in, len(pool)), size=min(3, len(pool) - n_in), replace=False)
    return [pool[-1]] + [pool[i] for i in picks], inputs, values


@pytest.mark.parametrize("seed", range(1000, 1100))
def test_view_graphs_evaluate_on_the_oracle(seed):
    results, inputs, values = build_views(seed)
    run("cpu", results, inputs, values)


def _lower_without_a_device(results, inputs):
    """Plan and lower every kernel of the computation with the dry-run runtime: whatever the
    planner groups, the lowering must be able to express (no GPU involved)."""
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    try:
        f = t.computation(results, *inputs)
        t.initialize()
        for kernel in t.kernel_groups[f].kernels:
            kernel.bind_buffers()
    finally:
        t.close()


# 6789: a reduction over a length-1 axis (an elementwise assignment whose result is written out)
# next to a reduction over all axes of a permuted view
@pytest.mark.parametrize("seed", list(range(1000, 1400)) + [6789])
def test_view_graphs_lower_without_a_device(seed):
    results, inputs, _ = build_views(seed)
    _lower_without_a_device(results, inputs)


@pytest.mark.parametrize("seed", range(200, 500))
def test_graphs_lower_without_a_device(seed):
    results, inputs, _ = build(seed)
    _lower_without_a_device(results, inputs)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", list(range(1000, 1100)) + [6789])
def test_random_view_graph_matches_oracle(seed):
    results, inputs, values = build_views(seed)
    want = run("cpu", results, inputs, values)
    got = run("hipgpu", results, inputs, values)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        ok = np.isfinite(w)
        np.testing.assert_allclose(g[ok], w[ok], rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ third generator: state
def build_state(seed):
    """Sequences of assignments to a few variables (whole tensors and row windows), each value an
    expression of the variables' current contents and an input: in-place updates, reads after
    writes, writes after reads -- what the planner's hazard rules exist for."""
    rs = np.random.RandomState(seed)
    A = ng.make_axis(int(rs.choice([4, 16, 33])), name="sa%d" % seed)
    B = ng.make_axis(int(rs.choice([8, 64, 100])), name="sb%d" % seed)
    init = [rs.uniform(-1, 1, (A.length, B.length)).astype(np.float32) for _ in range(3)]
    variables = [ng.variable([A, B], initial_value=v) for v in init]
    x = ng.placeholder([A, B])
    xv = rs.uniform(-1, 1, (A.length, B.length)).astype(np.float32)

    def expr(depth=0):
        if depth > 2 or rs.rand() < 0.3:
            return variables[rs.randint(3)] if rs.rand() < 0.7 else x
        if rs.rand() < 0.4:
            return [ng.tanh, ng.negative, ng.absolute, lambda t: t * 0.5][rs.randint(4)](expr(depth + 1))
        return [ng.add, ng.subtract, ng.multiply, ng.maximum][rs.randint(4)](expr(depth + 1), expr(depth + 1))

    steps = []
    for _ in range(rs.randint(3, 9)):
        target = variables[rs.randint(3)]
        value = expr()
        if not hasattr(value, "axes") or len(value.axes) != 2:
            continue
        if rs.rand() < 0.3 and A.length >= 4:
            lo = int(rs.randint(0, A.length - 2))
            hi = int(rs.randint(lo + 1, A.length + 1))
            window = [slice(lo, hi), slice(None)]
            tgt = ng.tensor_slice(target, window)
            val = ng.cast_axes(ng.tensor_slice(value, window), tgt.axes)
            steps.append(ng.assign(tgt, val))
        else:
            steps.append(ng.assign(target, value))
    total = ng.sum(variables[0] + variables[1] * 2.0 + variables[2] * 3.0, out_axes=())
    return ng.sequential(steps + [total]), variables, x, xv


def run_state(backend, seed, **kwargs):
    prog, variables, x, xv = build_state(seed)
    t = ngt.make_transformer_factory(backend, **kwargs)()
    try:
        f = t.computation(prog, x)
        read = t.computation([v * 1.0 for v in variables])
        totals = [np.array(f(xv)).copy(), np.array(f(xv * 0.5)).copy()]
        return totals, [np.array(r) for r in read()]
    finally:
        t.close()


@pytest.mark.parametrize("seed", range(2000, 2060))
def test_state_programs_evaluate_on_the_oracle(seed):
    run_state("cpu", seed)


@pytest.mark.gpu
@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "unfused"])
@pytest.mark.parametrize("seed", range(2000, 2060))
def test_random_state_program_matches_oracle(seed, fusion):
    want_tot, want_vars = run_state("cpu", seed)
    got_tot, got_vars = run_state("hipgpu", seed, fusion=fusion)
    for g, w in zip(got_vars, want_vars):
        np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-5)
    for g, w in zip(got_tot, want_tot):
        np.testing.assert_allclose(g, w, rtol=1e-4, atol=1e-3)


# ------------------------------------------------------------------ flex: host-managed vs device-resident
@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(120))
def test_flex_random_graph_host_and_device_management_agree(seed):
    """The same flex graph run three times with growing inputs under host-managed and under
    device-resident exponent management: results (dequantised values) must agree bit for bit,
    call after call."""
    def run_flex(resident):
        results, inputs, values = build(seed)
        t = ngt.make_transformer_factory("flexhip", resident=resident)()
        try:
            f = t.computation(results, *inputs)
            out = []
            for gain in (1.0, 3.0, 0.25):
                out.append([np.array(r).copy() for r in f(*[v * np.float32(gain) for v in values])])
            return out
        finally:
            t.close()

    host, device = run_flex(False), run_flex(True)
    for call, (h, d) in enumerate(zip(host, device)):
        for a, b in zip(h, d):
            np.testing.assert_array_equal(a, b, err_msg="call %d" % call)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(2000, 2050))
def test_flex_state_program_host_and_device_management_agree(seed):
    """Assignment programs (in-place updates keep their exponent for the kernel that reads and
    writes them) under both management modes: identical variables after two calls."""
    def run_flex(resident):
        prog, variables, x, xv = build_state(seed)
        t = ngt.make_transformer_factory("flexhip", resident=resident)()
        try:
            f = t.computation(prog, x)
            read = t.computation([v * 1.0 for v in variables])
            totals = [np.array(f(xv)).copy(), np.array(f(xv * 4.0)).copy(), np.array(f(xv * 0.1)).copy()]
            return totals, [np.array(r) for r in read()]
        finally:
            t.close()

    (h_tot, h_vars), (d_tot, d_vars) = run_flex(False), run_flex(True)
    for a, b in zip(h_vars, d_vars):
        np.testing.assert_array_equal(a, b)
    for a, b in zip(h_tot, d_tot):
        np.testing.assert_array_equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(1000, 1040))
def test_flex_view_graph_host_and_device_management_agree(seed):
    def run_flex(resident):
        results, inputs, values = build_views(seed)
        t = ngt.make_transformer_factory("flexhip", resident=resident)()
        try:
            f = t.computation(results, *inputs)
            return [[np.array(r).copy() for r in f(*[v * np.float32(g) for v in values])] for g in (1.0, 2.5, 0.2)]
        finally:
            t.close()

    host, device = run_flex(False), run_flex(True)
    for h, d in zip(host, device):
        for a, b in zip(h, d):
            np.testing.assert_array_equal(a, b)


# ------------------------------------------------------------------ the planner's large-tensor rules on small graphs
@pytest.fixture
def everything_is_large(monkeypatch):
    """Repeating a producer chain in a later kernel and folding a small kernel into its consumers
    are rules for tensors above a size threshold, which the generators' shapes stay below.  With
    the threshold at a few elements the same rules apply to these graphs."""
    import ngraph_hip.transformers.hiptransform as ht
    monkeypatch.setattr(ht.FusionPlanner, "small_tensor", 6)


@pytest.mark.parametrize("seed", range(300))
def test_graphs_lower_without_a_device_under_large_tensor_rules(seed, everything_is_large):
    for builder in (build, build_views):
        results, inputs, _ = builder(seed)
        _lower_without_a_device(results, inputs)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(150))
def test_random_graphs_match_oracle_under_large_tensor_rules(seed, everything_is_large):
    results, inputs, values = build(seed)
    for g, w in zip(run("hipgpu", results, inputs, values), run("cpu", results, inputs, values)):
        np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-5)
    results, inputs, values = build_views(seed)
    for g, w in zip(run("hipgpu", results, inputs, values), run("cpu", results, inputs, values)):
        ok = np.isfinite(w)
        np.testing.assert_allclose(g[ok], w[ok], rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(500, 650))
def test_state_programs_match_oracle_under_large_tensor_rules(seed, everything_is_large):
    """Moving a computation into a later kernel must respect every write in between: an
    assignment to a window of a variable the moved ops read, a kernel iterating over a window
    of the moved op's axes."""
    want_tot, want_vars = run_state("cpu", seed)
    got_tot, got_vars = run_state("hipgpu", seed)
    for g, w in zip(got_vars, want_vars):
        np.testing.assert_allclose(g, w, rtol=2e-5, atol=2e-5)
    for g, w in zip(got_tot, want_tot):
        np.testing.assert_allclose(g, w, rtol=1e-4, atol=1e-3)
