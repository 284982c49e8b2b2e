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
