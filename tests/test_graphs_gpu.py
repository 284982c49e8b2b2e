"""The launches of a small computation recorded as one HIP graph and replayed.

A graph is replayed several times, with the program's own eager work (host writes of new
inputs, reads of the results, synchronisations) between the replays, and every replay is
checked against the oracle and against the launches made one by one.
"""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from ngraph_hip.runtime.hiplib import FusedSpecBuilder, HipLibraryError
from oracle import configs, numpy_ops

pytestmark = pytest.mark.gpu
f32 = np.float32
RTOL, ATOL = 1e-5, 1e-6


def test_two_independent_launches_side_by_side_and_a_dependent_one(hip_runtime):
    """C ABI: y = tanh(x) and z = x * x recorded side by side, then w = y + z after the join;
    six replays with new x written in between."""
    rt = hip_runtime
    n = 1 << 16
    x_d, y_d, z_d, w_d = (rt.empty((n,)) for _ in range(4))

    def spec(build):
        sb = FusedSpecBuilder([n])
        build(sb)
        return sb.build()

    def s_tanh(sb):
        sb.store(sb.tensor(y_d.ptr, [1]), sb.unary("tanh", sb.load(sb.tensor(x_d.ptr, [1]))))

    def s_sqr(sb):
        r = sb.load(sb.tensor(x_d.ptr, [1]))
        sb.store(sb.tensor(z_d.ptr, [1]), sb.binary("mul", r, r))

    def s_add(sb):
        sb.store(sb.tensor(w_d.ptr, [1]), sb.binary("add", sb.load(sb.tensor(y_d.ptr, [1])), sb.load(sb.tensor(z_d.ptr, [1]))))

    specs = [spec(s_tanh), spec(s_sqr), spec(s_add)]
    rs = np.random.RandomState(1)
    x = rs.normal(0, 1, n).astype(f32)
    x_d.set(x)
    for s in specs:                      # once without recording: whatever a launch allocates exists afterwards
        rt.launch_fused(s)
    rt.sync()
    rt.graph_begin()
    rt.graph_fork()
    rt.launch_fused(specs[0])
    rt.graph_side(True)
    rt.launch_fused(specs[1])
    rt.graph_join()
    rt.launch_fused(specs[2])
    graph = rt.graph_end()
    assert rt.graph_nodes(graph) >= 3
    try:
        for i in range(6):
            x = rs.normal(0, 1 + i, n).astype(f32)
            x_d.set(x)
            for d in (y_d, z_d, w_d):
                d.set(np.full(n, np.nan, f32))        # a replay that skipped a launch would show
            rt.graph_launch(graph)
            want = numpy_ops.binary("add", numpy_ops.unary("tanh", x), numpy_ops.binary("mul", x, x))
            np.testing.assert_allclose(w_d.get(), want, rtol=RTOL, atol=ATOL, err_msg="replay %d" % i)
            np.testing.assert_array_equal(z_d.get(), x * x)
    finally:
        rt.graph_free(graph)
        for d in (x_d, y_d, z_d, w_d):
            d.free()


def test_recording_needs_an_open_capture(hip_runtime):
    rt = hip_runtime
    for call in (rt.graph_fork, rt.graph_join, lambda: rt.graph_side(True), rt.graph_end):
        with pytest.raises(HipLibraryError):
            call()
    rt.graph_begin()
    with pytest.raises(HipLibraryError):
        rt.graph_begin()
    with pytest.raises(HipLibraryError):
        rt.graph_side(True)                    # no fork is open
    rt.graph_abandon()
    rt.sync()                                  # the context works as before


def test_a_launch_whose_buffers_would_have_to_grow_is_refused_while_recording():
    """A split reduction takes a workspace the context allocates at its first such launch; in a
    fresh context that first launch cannot be a recorded one (growing would synchronise the
    stream, and the graph would keep an address).  The refusal leaves the context usable: the
    same launch made once outside a recording can then be recorded."""
    from ngraph_hip.runtime import HipRuntime
    rt = HipRuntime(0)
    try:
        R, A = 1 << 20, 4
        x = np.random.RandomState(2).uniform(0.5, 1.5, (R, A)).astype(f32)
        x_d, out_d = rt.array(x), rt.empty((A,))
        sb = FusedSpecBuilder([R, A])
        sb.reduce("sum", sb.load(sb.tensor(x_d.ptr, [A, 1])), sb.tensor(out_d.ptr, [0, 1]))
        spec = sb.build()
        rt.graph_begin()
        with pytest.raises(HipLibraryError, match="while a graph is being recorded"):
            rt.launch_fused(spec)
        rt.graph_abandon()
        rt.launch_fused(spec)
        want = numpy_ops.reduce("sum", x, 0)
        np.testing.assert_allclose(out_d.get(), want, rtol=1e-5)
        rt.graph_begin()
        rt.launch_fused(spec)
        graph = rt.graph_end()
        for i in range(3):
            out_d.set(np.full(A, np.nan, f32))
            rt.graph_launch(graph)
            np.testing.assert_allclose(out_d.get(), want, rtol=1e-5, err_msg="replay %d" % i)
        rt.graph_free(graph)
        x_d.free()
        out_d.free()
    finally:
        rt.close()


def _lstm_computation(t, Hn, Nn):
    H, N, G = ng.make_axis(Hn, name="H"), ng.make_axis(Nn, name="N"), ng.make_axis(4 * Hn, name="G")
    gates_st, cprev_st = ng.placeholder([N, G]), ng.placeholder([N, H])
    gates = ng.axes_with_order(gates_st, [G, N])
    c_prev = ng.axes_with_order(cprev_st, [H, N])
    parts = {k: ng.cast_axes(ng.tensor_slice(gates, [slice(j * Hn, (j + 1) * Hn), slice(None)]), [H, N])
             for j, k in enumerate(("i", "f", "o", "g"))}
    h, c = neon.lstm_cell(parts, c_prev, H, None)
    db = ng.sum(gates, out_axes=[G])
    return t.computation([c, h, db], gates_st, cprev_st)


@pytest.mark.parametrize("Hn,Nn", [(1024, 64), (96, 7)])
def test_lstm_cell_and_bias_gradient_replayed_as_one_graph(Hn, Nn):
    """The LSTM cell and the column sum for its bias gradient are two kernels that touch no
    common result: with graphs=True they are recorded side by side after two ordinary executions
    and replayed; every call, before and after, gives the oracle's results."""
    t = ngt.make_transformer_factory("hipgpu", graphs=True)()
    try:
        f = _lstm_computation(t, Hn, Nn)
        group = None
        for i in range(7):
            gates_np, cprev_np = configs.c4_inputs(Hn, Nn, seed=3 + i)
            c_w, h_w, db_w = configs.c4_cpu(gates_np, cprev_np)
            c_g, h_g, db_g = f(gates_np, cprev_np)
            group = t.kernel_groups[f]
            np.testing.assert_allclose(c_g, c_w, rtol=RTOL, atol=ATOL, err_msg="call %d" % i)
            np.testing.assert_allclose(h_g, h_w, rtol=RTOL, atol=ATOL, err_msg="call %d" % i)
            np.testing.assert_allclose(db_g, db_w, rtol=RTOL, atol=1e-5, err_msg="call %d" % i)
            assert (group._graph is not None) == (i >= group.graph_after_calls - 1), i
        assert t.runtime.graph_nodes(group._graph) >= 2
    finally:
        t.close()


def test_graphs_are_off_by_default_and_large_kernels_are_left_alone(monkeypatch):
    monkeypatch.delenv("NGH_GRAPHS", raising=False)
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        f = _lstm_computation(t, 96, 7)
        for i in range(4):
            f(*configs.c4_inputs(96, 7, seed=i))
        assert t.kernel_groups[f]._graph is None
    finally:
        t.close()
    monkeypatch.setenv("NGH_GRAPHS", "1")
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        f = _lstm_computation(t, 96, 7)
        for i in range(4):
            f(*configs.c4_inputs(96, 7, seed=i))
        assert t.kernel_groups[f]._graph is not None
    finally:
        t.close()
    t = ngt.make_transformer_factory("hipgpu", graphs=True)()
    try:
        A, B = ng.make_axis(2048, name="A"), ng.make_axis(2048, name="B")
        x = ng.placeholder([A, B])
        m = ng.max(x, out_axes=[A])
        f = t.computation([ng.exp(x - m), m], x)
        x_np = np.random.RandomState(0).normal(0, 1, (2048, 2048)).astype(f32)
        for i in range(4):
            f(x_np)
        assert t.kernel_groups[f]._graph is None          # 4 M elements per kernel: not launch-bound
    finally:
        t.close()


def test_a_computation_with_random_fills_is_not_recorded():
    """A random fill draws new numbers in every execution (a counter among its arguments): its
    launches are not recorded."""
    t = ngt.make_transformer_factory("hipgpu", graphs=True)()
    try:
        A = ng.make_axis(4096, name="A")
        x = ng.placeholder([A])
        y = x * ng.uniform(ng.temporary([A]), 0.0, 1.0)
        f = t.computation([y, ng.sum(y, out_axes=[])], x)
        seen = [np.array(f(np.ones(4096, f32))[0]).copy() for _ in range(5)]
        assert t.kernel_groups[f]._graph is None
        assert not np.array_equal(seen[3], seen[4])
    finally:
        t.close()
