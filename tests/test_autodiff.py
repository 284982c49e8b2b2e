"""Derivatives of elementwise ops, reductions and views: the backward graphs are ordinary
fused kernels.  Symbolic derivatives are checked against one-sided numeric ones the way
tests/transformer_dependent/test_execution.py does (:185-206 reductions, :336-346 reciprocal,
:414-445 and :448-469 elementwise, :471-533 broadcasting operands, :600-620 and :816-860 cross
entropies, :765-783 softmax, :899-916 sigmoid, :1074-1150 mean / variance, :1191-1205 broadcast),
and test_reshaping.py (:31-98 expand_dims, :100-171 slices, :190-230 overlapping slices, :298-327
cast_axes), test_ssa.py:111-151 (slice derivatives).
"""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.testing import executor, ExecutorFactory, RandomTensorGenerator, check_derivative
import oracle.cpu_transformer  # noqa: F401

rng = RandomTensorGenerator(0, np.float32)
BACKENDS = ["cpu", pytest.param("hipgpu", marks=pytest.mark.gpu),
            pytest.param("hipgpu-nofuse", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    name = request.param
    factory = (ngt.make_transformer_factory("hipgpu", fusion=False) if name == "hipgpu-nofuse"
               else ngt.make_transformer_factory(name))
    ngt.set_transformer_factory(factory)
    yield name
    ngt.set_transformer_factory(None)


def _input(rec=False):
    axes = [ng.make_axis(3), ng.make_axis(4, name="N")] + ([ng.make_axis(4, name="REC")] if rec else [])
    return ng.placeholder(axes)


def test_a_tensor_needs_an_error_and_unconnected_is_zero():
    p = ng.placeholder([ng.make_axis(5)])
    with pytest.raises(ValueError):
        ng.deriv(p, p)
    q = ng.placeholder([ng.make_axis(5)])
    zero = ng.deriv(ng.sum(p, out_axes=()), q)
    assert zero.axes == q.axes and zero.forwarded.is_constant


@pytest.mark.parametrize("reduction", ["sum", "prod"])
@pytest.mark.parametrize("sub", [slice(0, 1), slice(1, 2), slice(2, 3), slice(0, 2), slice(1, 3), slice(0, 3)])
def test_reduction_deriv(backend, reduction, sub):
    axes = ng.make_axes([ng.make_axis(4), ng.make_axis(5), ng.make_axis(3)])
    u = rng.discrete_uniform(1.0, 2.0, 0.002, axes) if hasattr(rng, "discrete_uniform") \
        else np.round(rng.uniform(1.0, 2.0, axes) / 0.002) * 0.002
    if reduction == "prod":
        u = (1.0 + (u - 1.0) * 0.25).astype(np.float32)         # keep products of 60 factors small
    p_u = ng.placeholder(axes)
    check_derivative(getattr(ng, reduction)(p_u, reduction_axes=axes[sub]), p_u, 0.001, u.astype(np.float32),
                     atol=1e-1, rtol=1e-1)


def test_max_min_deriv_picks_the_extremum(backend):
    x = _input()
    xv = np.arange(12, dtype=np.float32).reshape(3, 4) * np.float32(0.37) % np.float32(2.0)
    for red, np_arg in ((ng.max, np.argmax), (ng.min, np.argmin)):
        f = ng.sum(red(x, out_axes=[x.axes[1]]), out_axes=())
        with executor(ng.deriv(f, x), x) as g:
            got = g(xv)
        want = np.zeros_like(xv)
        want[np_arg(xv, axis=0), np.arange(4)] = 1
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("op", ["add", "subtract", "multiply", "divide", "maximum", "minimum", "power"])
def test_elementwise_binary_deriv(backend, op):
    axes = ng.make_axes([ng.make_axis(5), ng.make_axis(4)])
    p_u, p_v = ng.placeholder(axes), ng.placeholder(axes)
    u, v = rng.uniform(1.0, 2.0, axes), rng.uniform(2.5, 3.5, axes)     # no ties, no zeros
    f = getattr(ng, op)(p_u, p_v)
    check_derivative(f, p_u, 0.001, u, parameters=[p_v], parameter_values=[v], atol=2e-2, rtol=2e-2)
    check_derivative(f, p_v, 0.001, v, parameters=[p_u], parameter_values=[u], atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("op", ["exp", "log", "tanh", "reciprocal", "sqrt", "square", "negative", "absolute",
                                "sin", "cos", "sigmoid", "sigmoidAtomic", "safelog"])
def test_elementwise_unary_deriv(backend, op):
    axes = ng.make_axes([ng.make_axis(5), ng.make_axis(4)])
    p_u = ng.placeholder(axes)
    u = rng.uniform(0.5, 2.0, axes)
    check_derivative(getattr(ng, op)(p_u), p_u, 0.001, u, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("op", ["add", "subtract", "multiply", "divide"])
def test_elementwise_deriv_with_broadcast_operands(backend, op):
    W, H, N = ng.make_axis(2), ng.make_axis(3), ng.make_axis(4, name="N")
    p_u, p_v = ng.placeholder([W, H]), ng.placeholder([H, N])           # result has W, H, N
    u, v = rng.uniform(1.0, 2.0, p_u.axes), rng.uniform(1.0, 2.0, p_v.axes)
    for f in (getattr(ng, op)(p_u, p_v), getattr(ng, op)(p_v, p_u)):
        check_derivative(f, p_u, 0.001, u, parameters=[p_v], parameter_values=[v], atol=2e-2, rtol=2e-2)
        check_derivative(f, p_v, 0.001, v, parameters=[p_u], parameter_values=[u], atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("rec", [False, True])
def test_softmax_and_cross_entropy_deriv(backend, rec):
    p_x = _input(rec)
    p_t = ng.placeholder(p_x.axes)
    x = rng.uniform(0, 1, p_x.axes)
    e = np.exp(rng.uniform(0, 1, p_t.axes))
    t = (e / e.sum(axis=0, keepdims=True)).astype(np.float32)
    check_derivative(ng.softmax(p_x), p_x, 0.001, x, atol=1e-2, rtol=1e-2)
    check_derivative(ng.cross_entropy_multi(ng.softmax(p_x), p_t), p_x, 0.001, x,
                     parameters=[p_t], parameter_values=[t], atol=1e-2, rtol=1e-2)


def test_sigmoid_and_binary_cross_entropy_deriv(backend):
    p_u = _input()
    p_v = ng.placeholder(p_u.axes)
    u, v = rng.uniform(-3.0, 3.0, p_u.axes), rng.uniform(-3.0, 3.0, p_u.axes)
    check_derivative(ng.sigmoid(p_u), p_u, 0.001, u, atol=1e-2, rtol=1e-2)
    check_derivative(ng.log(ng.sigmoid(p_u)), p_u, 0.001, u, atol=1e-2, rtol=1e-2)
    val = ng.cross_entropy_binary_inner(ng.sigmoid(p_u), ng.softmax(p_v))
    check_derivative(val, p_u, 0.001, u, parameters=[p_v], parameter_values=[v], atol=1e-2, rtol=1e-2)


def test_variance_and_batch_norm_statistics_wgrad(backend):
    inputs = _input()
    targets = ng.placeholder(inputs.axes)
    xv, tv = rng.uniform(-0.1, 0.1, inputs.axes), rng.uniform(-0.1, 0.1, inputs.axes)
    var = ng.variance(inputs, reduction_axes=inputs.axes.batch_axes())
    err = ng.sum(var - targets, out_axes=())
    with executor([err, ng.deriv(err, inputs)], inputs, targets) as f:
        fwd, bwd = f(xv, tv)
    np.testing.assert_allclose(fwd, np.sum(np.var(xv, axis=1, keepdims=True) - tv), atol=1e-4, rtol=1e-4)
    # (each of the N targets sees the variance once, so the 1/N of the variance cancels)
    np.testing.assert_allclose(bwd, 2 * (xv - xv.mean(axis=1, keepdims=True)), atol=1e-4, rtol=1e-4)

    xv, tv = rng.uniform(-1, 1, inputs.axes), rng.uniform(-1, 1, inputs.axes)
    stat = ng.reciprocal(ng.sqrt(ng.variance(inputs, reduction_axes=inputs.axes.batch_axes()) + 1e-3))
    err = ng.sum(stat - targets, out_axes=())
    with executor([err, ng.deriv(err, inputs)], inputs, targets) as f:
        fwd, bwd = f(xv, tv)
    npv = np.var(xv, axis=1, keepdims=True) + 1e-3
    np_stat = 1.0 / np.sqrt(npv)
    np.testing.assert_allclose(fwd, np.sum(np_stat - tv), atol=1e-4, rtol=1e-4)
    np.testing.assert_allclose(bwd, -0.5 * np_stat / npv * 2 * (xv - xv.mean(axis=1, keepdims=True)),
                               atol=1e-4, rtol=1e-4)


def test_broadcast_deriv_reorder(backend):
    H, W = ng.make_axis(2), ng.make_axis(3)
    x = ng.constant(np.random.RandomState(0).rand(2, 3), axes=[H, W])
    dx = ng.deriv(ng.sum(ng.broadcast(x, [W, H]), out_axes=()), x)
    with executor(dx) as f:
        np.testing.assert_allclose(f(), np.ones((2, 3)))


@pytest.mark.parametrize("tensor,s", [([[1, 3], [2, 5]], [0, 1]), ([[1, 3], [2, 5]], [slice(None), 0]),
                                      ([[1, 3], [2, 5]], [1, slice(None)]), ([[1, 4, 5], [2, 5, 6]], [1, slice(1, 3)])])
def test_slice_deriv(backend, tensor, s):
    data = np.array(tensor, dtype=np.float32)
    x = ng.placeholder([ng.make_axis(n) for n in data.shape])
    check_derivative(ng.tensor_slice(x, s), x, 0.001, data, atol=1e-2, rtol=1e-2)


def test_overlapping_slices_deriv(backend):
    C, D = ng.make_axis(2), ng.make_axis(3)
    x = ng.placeholder([C, D])
    x_np = np.array([[10, 20, 30], [1, 2, 3]], dtype=np.float32)
    y1 = x[0, :] * 2 + x[1, :] * 3
    y2 = x[0, :] * 2 + x[1, :] * 3 + 4 * x[1, :]
    for y in (y1, y2):
        check_derivative(y, x, 0.01, x_np, atol=5e-2, rtol=1e-2)
    with ExecutorFactory() as ex:                       # known answer of test_ssa.py:134-151
        got = ex.derivative(x[0, :] + x[1, :], x)(x_np)
    want = np.zeros((3, 2, 3), np.float32)
    for i in range(3):
        want[i, :, i] = 1
    np.testing.assert_allclose(got, want)


def test_expand_dims_and_cast_axes_deriv(backend):
    data = np.array([[2, 5], [13, 5]], dtype=np.float32)
    for dim in range(3):
        x = ng.placeholder([ng.make_axis(2), ng.make_axis(2)])
        check_derivative(ng.expand_dims(x, ng.make_axis(3), dim), x, 0.001, data, atol=1e-2, rtol=1e-2)
    C, D = ng.make_axis(2), ng.make_axis(3)
    x = ng.placeholder([C, D])
    y = x + ng.cast_axes(x[1, :], [D])
    check_derivative(y, x, 0.01, np.array([[10, 20, 30], [1, 2, 3]], dtype=np.float32), atol=5e-2, rtol=1e-2)


def test_a_training_step_built_from_deriv(backend):
    """Logistic regression on a fixed design without a dense op: weights broadcast over the batch,
    the gradient comes from deriv, the update is an assignment -- forward, backward and update all
    run as fused kernels.  Checked against the closed form of the gradient."""
    F, N = ng.make_axis(6, name="F"), ng.make_axis(16, name="N")
    rs = np.random.RandomState(2)
    xv, tv, w0 = rs.normal(0, 1, (6, 16)).astype(np.float32), rs.randint(0, 2, 16).astype(np.float32), \
        rs.normal(0, 0.1, 6).astype(np.float32)
    x, t = ng.placeholder([F, N]), ng.placeholder([N])
    w = ng.variable([F], initial_value=w0)
    y = ng.sigmoid(ng.sum(w * x, out_axes=[N]))
    loss = ng.sum(ng.cross_entropy_binary_inner(y, t), out_axes=()) / 16.0
    grad = ng.deriv(loss, w)
    step = ng.sequential([ng.assign(w, w - 0.5 * grad), loss])
    with executor(step, x, t) as f:
        losses = [float(f(xv, tv)) for _ in range(5)]
    wn = w0.astype(np.float64)
    want = []
    for _ in range(5):
        p = 1.0 / (1.0 + np.exp(-(wn[:, None] * xv).sum(axis=0)))
        want.append(float(np.mean(-(tv * np.log(p) + (1 - tv) * np.log(1 - p)))))
        wn = wn - 0.5 * (xv * (p - tv)).sum(axis=1) / 16.0
    np.testing.assert_allclose(losses, want, rtol=2e-5)
    assert losses[-1] < losses[0]


def test_batch_norm_backward_closed_form(backend):
    """neon.batch_norm_train differentiates itself as a whole (two reductions in one pass, one
    elementwise pass); checked against the textbook formulas in float64 and against numeric
    derivatives of the op-by-op composite."""
    from ngraph_hip.frontends import neon
    C, H, N = ng.make_axis(4, name="C"), ng.make_axis(5, name="H"), ng.make_axis(6, name="N")
    x, e = ng.placeholder([C, H, N]), ng.placeholder([C, H, N])
    gv = np.array([1.0, 2.0, 0.5, 1.5], np.float32)
    g, b = ng.variable([C], initial_value=gv), ng.variable([C], initial_value=np.zeros(4, np.float32))
    y, _, _ = neon.batch_norm_train(x, g, b, [C])
    rs = np.random.RandomState(0)
    xv, ev = rs.normal(0.5, 2, (4, 5, 6)).astype(np.float32), rs.normal(0, 1, (4, 5, 6)).astype(np.float32)
    with executor([ng.deriv(y, x, error=e), ng.deriv(y, g, error=e), ng.deriv(y, b, error=e)], x, e) as f:
        dx, dg, db = f(xv, ev)
    x64, e64 = xv.reshape(4, -1).astype(np.float64), ev.reshape(4, -1).astype(np.float64)
    rstd = 1 / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    xh = (x64 - x64.mean(1, keepdims=True)) * rstd
    dg_want, db_want = (e64 * xh).sum(1), e64.sum(1)
    dx_want = gv[:, None] * rstd * (e64 - db_want[:, None] / 30 - xh * dg_want[:, None] / 30)
    np.testing.assert_allclose(dx.reshape(4, -1), dx_want, rtol=1e-4, atol=2e-6)
    np.testing.assert_allclose(dg, dg_want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, db_want, rtol=1e-5, atol=1e-5)
    # the same layer written out op by op, differentiated rule by rule
    flat_mean = ng.mean(x, out_axes=[C])
    flat_var = ng.variance(x, out_axes=[C])
    y_plain = g * ((x - flat_mean) * ng.reciprocal(ng.sqrt(flat_var + 1e-5))) + b
    with executor(ng.deriv(y_plain, x, error=e), x, e) as f:
        np.testing.assert_allclose(f(xv, ev), dx, rtol=1e-3, atol=1e-5)


def test_recomputation_replaces_a_round_trip_through_memory():
    """Planner property, no GPU: the normalised input of the batch-norm backward is needed by the
    reduction kernel and by the elementwise kernel after it; the second recomputes it from x
    instead of reading a copy the first would have to write."""
    from ngraph_hip.frontends import neon
    from ngraph_hip.runtime.hiplib import OPCODES
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    try:
        C, R = ng.make_axis(16, name="C"), ng.make_axis(16384, name="R")
        x, e = ng.placeholder([C, R]), ng.placeholder([C, R])
        g, b = ng.variable([C], initial_value=1.0), ng.variable([C], initial_value=0.0)
        y, _, _ = neon.batch_norm_train(x, g, b, [C])
        f = t.computation([ng.deriv(y, x, error=e), ng.deriv(y, g, error=e), ng.deriv(y, b, error=e)], x, e)
        t.initialize()
        big_stores, kernels = 0, []
        for kernel in t.kernel_groups[f].kernels:
            kernel.bind_buffers()
            kernels.extend(getattr(kernel, "kernels", [kernel]))      # (a run of kernels: what it settled on)
        for kernel in kernels:
            for spec in getattr(kernel, "specs", []):
                if spec.shape[0] * spec.shape[1] * spec.shape[2] < 16 * 16384:
                    continue
                big_stores += sum(1 for i in range(spec.n_ops) if spec.ops[i].opcode == OPCODES["store"]
                                  and all(spec.tensors[spec.ops[i].dst].strides[a] != 0 or spec.shape[a] == 1
                                          for a in range(3)))
        assert big_stores == 1          # dx, and nothing else of that size
        # the per-channel factors between the passes (gamma * rstd, the two sums over m) are
        # repeated inside the dx kernel instead of costing launches of their own
        assert len(kernels) == 3     # statistics, the two sums, dx
    finally:
        t.close()


@pytest.mark.gpu
def test_per_channel_factors_absorbed_into_the_big_kernels():
    """Small elementwise kernels between passes over a large tensor are repeated inside their
    consumers (operands become broadcast loads); values against float64 closed forms, on axes
    that do not merge into one row axis."""
    from ngraph_hip.frontends import neon
    C, H, N = ng.make_axis(8, name="C"), ng.make_axis(48, name="H"), ng.make_axis(256, name="N")
    x, e = ng.placeholder([C, H, N]), ng.placeholder([C, H, N])
    rs = np.random.RandomState(3)
    gv = rs.uniform(0.5, 2, 8).astype(np.float32)
    g, b = ng.variable([C], initial_value=gv), ng.variable([C], initial_value=np.zeros(8, np.float32))
    y, _, _ = neon.batch_norm_train(x, g, b, [C])
    xv = rs.normal(0.5, 2, (8, 48, 256)).astype(np.float32)
    ev = rs.normal(0, 1, (8, 48, 256)).astype(np.float32)
    t = ngt.make_transformer_factory("hipgpu")()
    try:
        f = t.computation([ng.deriv(y, x, error=e), ng.deriv(y, g, error=e), ng.deriv(y, b, error=e)], x, e)
        # a per-channel scale feeding a large elementwise result and a reduction
        s = ng.variable([C], initial_value=gv)
        k = ng.sqrt(s * s + 1.0) * 0.5
        f2 = t.computation([x * k, ng.sum(e * k, out_axes=[C])], x, e)
        dx, dg, db = f(xv, ev)
        assert len(t.kernel_groups[f].kernels) == 3
        xs, es = f2(xv, ev)
        assert len(t.kernel_groups[f2].kernels) == 1      # the scale chain, x * k and the sum
    finally:
        t.close()
    m = 48 * 256
    x64, e64 = xv.reshape(8, -1).astype(np.float64), ev.reshape(8, -1).astype(np.float64)
    rstd = 1 / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    xh = (x64 - x64.mean(1, keepdims=True)) * rstd
    dg_want, db_want = (e64 * xh).sum(1), e64.sum(1)
    dx_want = gv[:, None] * rstd * (e64 - db_want[:, None] / m - xh * dg_want[:, None] / m)
    np.testing.assert_allclose(dx.reshape(8, -1), dx_want, rtol=1e-4, atol=2e-6)
    np.testing.assert_allclose(dg, dg_want, rtol=1e-5, atol=1e-3)
    np.testing.assert_allclose(db, db_want, rtol=1e-5, atol=1e-3)
    k64 = np.sqrt(gv.astype(np.float64) ** 2 + 1.0) * 0.5
    np.testing.assert_allclose(xs.reshape(8, -1), x64 * k64[:, None], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(es, (e64 * k64[:, None]).sum(1), rtol=1e-5, atol=1e-3)


# ---- stack / concat: assignments into slices of a temporary, on the device ---------------------
@pytest.mark.parametrize("pos", [0, 1, 2])
def test_stack_and_its_derivative(backend, pos):
    """test_stack_tensor.py:29-56: value against numpy.stack, symbolic against numeric derivative
    with respect to every argument."""
    W, H, I = ng.make_axis(4, name="W"), ng.make_axis(5, name="H"), ng.make_axis(3, name="I")
    axes = ng.make_axes([W, H])
    gen = RandomTensorGenerator(0, np.float32)
    a_v = [gen.uniform(0, 1, axes) for _ in range(I.length)]
    a = [ng.placeholder(axes) for _ in a_v]
    s = ng.stack(a, I, pos)
    with ExecutorFactory() as ex:
        value = ex.executor(s, *a)
        nums = [ex.numeric_derivative(s, p, 1e-3, *[q for q in a if q is not p]) for p in a]
        syms = [ex.derivative(s, p, *[q for q in a if q is not p]) for p in a]
        np.testing.assert_array_equal(value(*a_v), np.stack(a_v, axis=pos))
        for i, (num, sym) in enumerate(zip(nums, syms)):
            others = [v for j, v in enumerate(a_v) if j != i]
            np.testing.assert_allclose(num(a_v[i], *others), sym(a_v[i], *others), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("num_vars,num_axes,concat_pos", [(1, 2, 1), (2, 3, 2), (15, 5, 1)])
def test_concatenate_and_its_derivative(backend, num_vars, num_axes, concat_pos):
    """test_op_graph_transformer_dependent.py:25-42, 166-177."""
    rs = np.random.RandomState(num_vars)
    common = [ng.make_axis(2, name="c%d" % i) for i in range(num_axes - 1)]
    ax = ng.make_axis(int(rs.randint(3, 10)), name="cat")
    axes = ng.make_axes(common[:concat_pos] + [ax] + common[concat_pos:])
    np_list = [rs.uniform(0, 1, axes.lengths).astype(np.float32) for _ in range(num_vars)]
    x_list = [ng.constant(v, axes=axes) for v in np_list]
    with ExecutorFactory() as ex:
        v = ng.concat_along_axis(x_list, x_list[0].axes[concat_pos])
        d = ng.deriv(v, x_list[0], error=ng.constant(np.ones(v.axes.lengths, np.float32), axes=v.axes))
        e_v, e_d = ex.executor([v, d])()
        np.testing.assert_array_equal(e_v, np.concatenate(np_list, axis=concat_pos))
        np.testing.assert_array_equal(e_d, np.ones(axes.lengths))


def test_concat_different_axis_lengths_and_state(backend):
    """test_op_graph_transformer_dependent.py:180-196 (axes of one name, different lengths),
    test_ssa.py:93-106 (persistent tensors)."""
    ax1, ax2 = ng.make_axis(3, name="concat"), ng.make_axis(2, name="concat")
    ax3 = ng.make_axis(10, name="other")
    x, y = ng.placeholder([ax1, ax3]), ng.placeholder([ax2, ax3])
    rs = np.random.RandomState(0)
    np_x, np_y = rs.rand(3, 10).astype(np.float32), rs.rand(2, 10).astype(np.float32)
    A, B = ng.make_axis(3, name="A"), ng.make_axis(4, name="B")
    x0 = ng.persistent_tensor([A, B], initial_value=-np.ones((3, 4), np.float32))
    x1 = ng.persistent_tensor([A, B], initial_value=np.ones((3, 4), np.float32))
    with ExecutorFactory() as ex:
        f = ex.executor(ng.concat_along_axis([x, y], ax1), x, y)
        g = ex.executor(ng.concat_along_axis([x0, x1], A))
        np.testing.assert_array_equal(f(np_x, np_y), np.concatenate([np_x, np_y], axis=0))
        np.testing.assert_array_equal(g(), np.concatenate([-np.ones((3, 4)), np.ones((3, 4))], axis=0))
