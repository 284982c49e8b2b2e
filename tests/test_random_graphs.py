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
from oracle import error_bound
from graph_generators import build, build_views, build_state  # noqa: F401


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


def arbitrate(gen, seed, rtol=2e-5, atol=2e-5, **device_options):
    """Device and oracle against float64 with a running error bound (oracle/error_bound.py).
    Each of the three evaluations builds its own copy of the graph, so no rewrite one backend
    makes is seen by another.  Both float32 results must lie within tolerance + bound of the
    float64 value, element by element; an element where the oracle's own order of operations
    overflowed float32 (a long product passing through inf) binds neither side.  Returns the
    largest error of each side over the decided elements, for the record."""
    want = run("cpu", *gen(seed))
    got = run("hipgpu", *gen(seed), **device_options)
    results, inputs, values = gen(seed)
    t = ngt.make_transformer_factory("cpu_bound")()
    try:
        exact = [np.array(r) for r in t.computation(results, *inputs)(*values)]
        bounds = [t.error_bound(r) for r in results]
    finally:
        t.close()
    worst = [0.0, 0.0]
    for g, w, v, b in zip(got, want, exact, bounds):
        assert g.shape == w.shape == v.shape
        overflowed = ~np.isfinite(w)
        dev_ok = error_bound.within_bound(g, v, b, rtol, atol) | (overflowed & ~np.isfinite(g))
        ora_ok = error_bound.within_bound(w, v, b, rtol, atol) | overflowed
        assert ora_ok.all(), "oracle outside its own error bound at %s" % (np.argwhere(~ora_ok)[:3],)
        assert dev_ok.all(), "device outside the error bound at %s: %s, float64 %s, bound %s" % (
            np.argwhere(~dev_ok)[:3], g[~dev_ok][:3], v[~dev_ok][:3], b[~dev_ok][:3])
        decided = np.isfinite(b) & np.isfinite(v) & ~overflowed & np.isfinite(g)
        if decided.any():
            worst[0] = max(worst[0], float(np.abs(g[decided] - v[decided]).max()))
            worst[1] = max(worst[1], float(np.abs(w[decided] - v[decided]).max()))
    return worst


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
    arbitrate(build_views, seed)


# Every seed of 50 000 swept on the device (generator `build` 200-24199, `build_views`
# 1100-27099) whose result differs from the oracle's by more than rtol = atol = 2e-5 somewhere:
# products of up to 100 factors, squares of exponentials and differences of nearly equal sums
# (outputs of magnitude 1e7 to 1e32 whose last bits two float32 evaluations cannot share), and
# comparisons / argmax positions that a last-bit difference of an operand flips (error "x25000"
# = 0 against 1).  Arbitrated against float64: both sides are within the forward error bound of
# the graph on every one, fused and one kernel per op.
ILL_CONDITIONED_VIEW_SEEDS = [
    1243, 1506, 1917, 2189, 2359, 2478, 2929, 3628, 3698, 3906, 4300, 4648, 4686, 5858, 6383, 6438,
    6635, 8192, 8284, 8556, 9651, 9988, 11429, 11635, 12270, 12308, 12328, 12346, 12471, 12882,
    12976, 13565, 14576, 14667, 14845, 15106, 15436, 15881, 16146, 16191, 16262, 17009, 17158,
    17413, 17732, 18640, 19354, 19704, 20250, 20381, 20876, 21053, 21108, 21913, 21982, 22196,
    22444, 22510, 22987, 23155, 23393, 23446, 23506, 23751, 23756, 24024, 24084, 24421, 24509,
    25156, 25186, 25571, 25644, 26598,
    # a later sweep (`build` 30000-34050: none; `build_views` 30000-35367, and 40000-42999 with one
    # kernel per op) with the chain kernels, ragged rows and the pair launch in place
    30183, 30373, 30846, 32106, 32127, 32138, 32209, 32934, 33034, 33217, 33252, 33455, 33936,
    34690, 34699, 35129, 40648, 41076, 41229, 41651, 41933, 41952, 42104, 42334,
    43237]               # (from 587 graphs with every stage compiled at run time)
ILL_CONDITIONED_SEEDS = [19997]


@pytest.mark.gpu
@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "unfused"])
@pytest.mark.parametrize("seed", ILL_CONDITIONED_VIEW_SEEDS)
def test_ill_conditioned_view_graph_is_within_the_float64_error_bound(seed, fusion):
    arbitrate(build_views, seed, fusion=fusion)


@pytest.mark.gpu
@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "unfused"])
@pytest.mark.parametrize("seed", ILL_CONDITIONED_SEEDS + list(range(200, 260)))
def test_graph_is_within_the_float64_error_bound(seed, fusion):
    arbitrate(build, seed, fusion=fusion)


def test_error_bound_is_not_vacuous_on_a_well_conditioned_graph():
    """tanh(a*x + b) * sigmoid(x): the bound stays at a few dozen ulp of the result."""
    H = ng.make_axis(512, name="vac_h")
    x = ng.placeholder([H])
    y = ng.tanh(x * 0.7 + 0.1) * ng.sigmoid(x)
    xv = np.linspace(-4, 4, 512).astype(np.float32)
    t = ngt.make_transformer_factory("cpu_bound")()
    value = t.computation(y, x)(xv)
    bound = t.error_bound(y)
    want = run("cpu", [y], [x], [xv])[0]
    assert (bound <= 64 * 2.0 ** -24 * np.maximum(np.abs(value), 1e-3)).all()
    assert error_bound.within_bound(want, value, bound, 0, 0).all()


def test_error_bound_sees_cancellation_and_undecided_comparisons():
    """(x + 1e7) - 1e7 keeps one or two digits of x in float32: the bound must say so, and a
    comparison of the result with x is undecided wherever the bound reaches the difference."""
    H = ng.make_axis(64, name="canc_h")
    x = ng.placeholder([H])
    y = (x + 1e7) - 1e7
    c = ng.greater(y, x)
    xv = np.random.RandomState(5).uniform(1, 2, 64).astype(np.float32)
    t = ngt.make_transformer_factory("cpu_bound")()
    value, flag = t.computation([y, c], x)(xv)
    bound, flag_bound = t.error_bound(y), t.error_bound(c)
    np.testing.assert_array_equal(value, xv.astype(np.float64))
    want = run("cpu", [y], [x], [xv])[0]
    err = np.abs(want - value)
    assert err.max() > 0.1 and (err <= bound).all() and (bound < 4.0).all()
    assert np.isinf(flag_bound).all()


@pytest.mark.parametrize("seed", range(150))
def test_oracle_float32_lies_within_the_bound_of_the_float64_evaluation(seed):
    """Pins the bound evaluator from the CPU side: with no tolerance added, the float32 oracle
    result is inside the bound around the float64 value for both generators' graphs."""
    for gen in (build, build_views):
        want = run("cpu", *gen(seed))
        results, inputs, values = gen(seed + 0)
        t = ngt.make_transformer_factory("cpu_bound")()
        exact = [np.array(r) for r in t.computation(results, *inputs)(*values)]
        for w, v, r in zip(want, exact, results):
            ok = error_bound.within_bound(w, v, t.error_bound(r), 0, 0) | ~np.isfinite(w)
            assert ok.all()


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
