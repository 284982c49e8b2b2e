"""Graph-level parity: the same test bodies run on the NumPy oracle transformer
("cpu", always) and on the HIP transformer ("hipgpu", GPU box) and are checked
against NumPy expressions written here, the way the reference's
tests/transformer_dependent/test_execution.py and test_kernel_generator.py do.
"""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.testing import executor, RandomTensorGenerator
import oracle.cpu_transformer  # noqa: F401  registers "cpu"

rng = RandomTensorGenerator(0, np.float32)
RTOL, ATOL = 1e-5, 1e-6

BACKENDS = ["cpu", pytest.param("hipgpu", marks=pytest.mark.gpu),
            pytest.param("hipgpu-nofuse", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    name = request.param
    if name == "hipgpu-nofuse":
        factory = ngt.make_transformer_factory("hipgpu", fusion=False)
    else:
        factory = ngt.make_transformer_factory(name)
    ngt.set_transformer_factory(factory)
    yield name
    ngt.set_transformer_factory(None)


def axes(**kw):
    return ng.make_axes([ng.make_axis(length=v, name=k) for k, v in kw.items()])


def test_transformer_registry():
    assert "cpu" in ngt.transformer_choices()
    assert "hipgpu" in ngt.transformer_choices()
    assert "flexhip" in ngt.transformer_choices()
    with pytest.raises(ValueError):
        ngt.allocate_transformer("no-such-backend")
    f = ngt.make_transformer_factory("cpu")
    assert f.name == "cpu"


def test_scalar_constant_and_placeholder(backend):
    x = ng.placeholder(())
    with executor(x * 2 + 1, x) as f:
        for v in (0.0, 1.5, -3.25):
            np.testing.assert_allclose(f(v), np.float32(v) * 2 + 1, rtol=RTOL)


UNARY = [(ng.negative, np.negative), (ng.absolute, np.abs), (ng.exp, np.exp), (ng.tanh, np.tanh),
         (ng.square, np.square), (ng.sign, np.sign), (ng.sin, np.sin), (ng.cos, np.cos),
         (ng.sigmoid, lambda x: 1.0 / (1.0 + np.exp(-x))),
         (ng.sigmoidAtomic, lambda x: 1.0 / (1.0 + np.exp(-x)))]


@pytest.mark.parametrize("ng_fn,np_fn", UNARY)
def test_unary_elementwise(backend, ng_fn, np_fn):
    ax = axes(H=17, W=33)
    x = ng.placeholder(ax)
    xv = rng.uniform(-2, 2, ax)
    with executor(ng_fn(x), x) as f:
        np.testing.assert_allclose(f(xv), np_fn(xv), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("ng_fn,np_fn", [(ng.sqrt, np.sqrt), (ng.log, np.log),
                                         (ng.reciprocal, np.reciprocal), (ng.safelog, np.log)])
def test_unary_positive_domain(backend, ng_fn, np_fn):
    ax = axes(H=8, W=65)
    x = ng.placeholder(ax)
    xv = rng.uniform(0.1, 5, ax)
    with executor(ng_fn(x), x) as f:
        np.testing.assert_allclose(f(xv), np_fn(xv), rtol=RTOL, atol=ATOL)


def test_safelog_follows_the_reference_statement_sequence(backend):
    """ng.safelog(x, limit) = maximum(log(x + exp(limit)), limit) (op_graph.py:3070-3072): zero
    gives the limit, a value below exp(limit) gives about the limit, a negative value NaN."""
    xv = np.array([0.0, 1e-30, 1e-22, np.exp(-50.0), 1e-10, 0.5, 1.0, 7.25, 3e4, -1e-3, -2.0], np.float32)
    ax = axes(W=xv.size)
    x = ng.placeholder(ax)
    for limit in (-50.0, -10.0):
        with np.errstate(all="ignore"):
            t = np.add(xv, np.float32(np.exp(limit)), dtype=np.float32)
            want = np.maximum(np.log(t, dtype=np.float32), np.float32(limit))
        with executor(ng.safelog(x, limit), x) as f:
            got = f(xv)
        assert np.isnan(want[-2:]).all() and want[0] == np.float32(limit)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL, equal_nan=True)


BINARY = [(ng.add, np.add), (ng.subtract, np.subtract), (ng.multiply, np.multiply),
          (ng.divide, np.divide), (ng.maximum, np.maximum), (ng.minimum, np.minimum),
          (ng.equal, np.equal), (ng.not_equal, np.not_equal), (ng.greater, np.greater),
          (ng.less, np.less), (ng.greater_equal, np.greater_equal), (ng.less_equal, np.less_equal)]


@pytest.mark.parametrize("ng_fn,np_fn", BINARY)
def test_binary_elementwise_matched_axes(backend, ng_fn, np_fn):
    ax = axes(C=5, H=12, N=16)
    x, y = ng.placeholder(ax), ng.placeholder(ax)
    xv, yv = rng.uniform(-2, 2, ax), rng.uniform(-2, 2, ax)
    yv[::2] = xv[::2]
    with executor(ng_fn(x, y), x, y) as f:
        np.testing.assert_allclose(f(xv, yv), np_fn(xv, yv).astype(np.float32), rtol=RTOL, atol=ATOL)


def test_binary_broadcast_unmatched_axes(backend):
    """x[C,N] + y[N,H]: result axes C,N,H (op_graph.py:3159-3180)."""
    C, N, H = ng.make_axis(3, name="C"), ng.make_axis(4, name="N"), ng.make_axis(5, name="H")
    x, y = ng.placeholder([C, N]), ng.placeholder([N, H])
    z = x + y
    assert z.axes == ng.make_axes([C, N, H])
    xv, yv = rng.uniform(-1, 1, x.axes), rng.uniform(-1, 1, y.axes)
    with executor(z, x, y) as f:
        np.testing.assert_allclose(f(xv, yv), xv[:, :, None] + yv[None, :, :], rtol=RTOL)
    # y already has all the axes: result takes y's order
    w = ng.placeholder([H, N, C])
    assert (x * w).axes == w.axes


def test_power_floordiv_mod(backend):
    ax = axes(H=9, W=31)
    x, y = ng.placeholder(ax), ng.placeholder(ax)
    xv = np.round(rng.uniform(-9, 9, ax))
    yv = np.round(rng.uniform(1, 4, ax)) * np.where(rng.uniform(0, 1, ax) > 0.5, 1, -1)
    with executor([x // y, x % y, ng.power(ng.absolute(x) + 0.5, y)], x, y) as f:
        fd, md, pw = f(xv, yv)
    np.testing.assert_allclose(fd, np.floor_divide(xv, yv), rtol=RTOL)
    np.testing.assert_allclose(md, np.mod(xv, yv), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(pw, np.power(np.abs(xv) + np.float32(0.5), yv), rtol=RTOL)


REDUCTIONS = [(ng.sum, np.sum), (ng.max, np.max), (ng.min, np.min), (ng.prod, np.prod)]


@pytest.mark.parametrize("ng_fn,np_fn", REDUCTIONS)
@pytest.mark.parametrize("sub", [slice(0, 1), slice(1, 2), slice(2, 3), slice(0, 2), slice(1, 3),
                                 slice(0, 3)])
def test_reduction_axis_slices(backend, ng_fn, np_fn, sub):
    """Every contiguous subset of reduction axes (test_execution.py:144-181)."""
    ax = axes(C=4, H=6, W=10)
    x = ng.placeholder(ax)
    xv = rng.uniform(0.5, 1.5, ax)
    red = ax[sub]
    np_axes = tuple(ax.index(a) for a in red)
    with executor(ng_fn(x, reduction_axes=red), x) as f:
        np.testing.assert_allclose(f(xv), np_fn(xv, axis=np_axes), rtol=1e-5, atol=1e-5)


def test_reduction_out_axes_and_noncontiguous(backend):
    ax = axes(C=3, H=5, W=7, N=4)
    x = ng.placeholder(ax)
    xv = rng.uniform(-1, 1, ax)
    # reduce over H and N (not adjacent in memory): needs a host loop or strided reduction
    with executor(ng.sum(x, out_axes=ax[0:1] + ax[2:3]), x) as f:
        np.testing.assert_allclose(f(xv), xv.sum(axis=(1, 3)), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("ng_fn,np_fn", [(ng.sum, np.sum), (ng.prod, np.prod), (ng.max, np.max), (ng.min, np.min)])
def test_reduction_over_axes_that_are_not_adjacent(backend, ng_fn, np_fn):
    """[N, C, H, W] reduced over N, H and W keeping C (the batch-norm statistics of the N-major
    layout), over N and W, and over C and W: the reduced axes form two strided groups."""
    ax = axes(N=6, C=5, H=7, W=9)
    x = ng.placeholder(ax)
    xv = rng.uniform(0.8, 1.25, ax)
    keep = [(ax[1:2], (0, 2, 3)), (ax[1:3], (0, 3)), (ax[0:1] + ax[2:3], (1, 3))]
    with executor([ng_fn(x, out_axes=out) for out, _ in keep], x) as f:
        got = f(xv)
    for g, (_, reduced) in zip(got, keep):
        np.testing.assert_allclose(g, np_fn(xv, axis=reduced), rtol=1e-5, atol=1e-6)


def _kernels_lowered_for(results, placeholders, backend="hipgpu"):
    t = ngt.make_transformer_factory(backend, dry_run=True, jit=False)()
    try:
        f = t.computation(results, *placeholders)
        t.initialize()
        t.kernel_groups[f].bind()        # (runs of kernels settle which of them merge)
        return [type(k).__name__ for k in t.kernel_groups[f].kernels]
    finally:
        t.close()


def test_split_reductions_need_no_copy_of_the_operand():
    """Sum / prod / max / min over axes in two strided groups are taken group by group (one
    pass over the operand, then a small reduction); argmax, whose result is a position along the
    original axes, and flex tensors, which would round the intermediate, copy the operand into
    (reduced, kept) order first, as the reference does (layout_common.py:347-378)."""
    ax = axes(N=6, C=5, H=7, W=9)
    x = ng.placeholder(ax)
    keep_c = ax[1:2]
    for fn in (ng.sum, ng.prod, ng.max, ng.min):
        assert "CopyKernel" not in _kernels_lowered_for([fn(x, out_axes=keep_c)], [x]), fn.__name__
    flat = ng.flatten_at(ng.axes_with_order(x, ax[0:1] + ax[2:4] + ax[1:2]), 3)
    assert "CopyKernel" in _kernels_lowered_for([ng.argmax(flat, out_axes=flat.axes[1:])], [x])
    assert "FlexCopyKernel" in _kernels_lowered_for([ng.sum(x, out_axes=keep_c)], [x], backend="flexhip")


def test_argmax_argmin_first_index_wins(backend):
    ax = axes(C=7, N=9)
    x = ng.placeholder(ax)
    xv = np.round(rng.uniform(-3, 3, ax))          # many ties
    with executor([ng.argmax(x, out_axes=ax[1:]), ng.argmin(x, out_axes=ax[1:])], x) as f:
        amax, amin = f(xv)
    np.testing.assert_array_equal(amax, xv.argmax(axis=0))
    np.testing.assert_array_equal(amin, xv.argmin(axis=0))


def test_mean_variance(backend):
    ax = axes(C=6, H=20, N=8)
    x = ng.placeholder(ax)
    xv = rng.normal(0.5, 2, ax)
    out = ax[0:1]
    with executor([ng.mean(x, out_axes=out), ng.variance(x, out_axes=out)], x) as f:
        m, v = f(xv)
    np.testing.assert_allclose(m, xv.mean(axis=(1, 2)), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v, xv.var(axis=(1, 2)), rtol=1e-5, atol=1e-6)


def test_mean_variance_over_axes_in_two_groups(backend):
    """Batch-norm statistics of an [N, C, H, W] tensor: mean and variance over N, H and W, then
    the normalisation.  The HIP transformer takes one-pass moments of the H*W rows and combines
    them over N (mean of the rows' means; mean of the rows' variances plus the squared distance
    of their means), which is exact for rows of equal length."""
    ax = axes(N=6, C=5, H=16, W=8)
    x = ng.placeholder(ax)
    gamma, beta = ng.placeholder(ax[1:2]), ng.placeholder(ax[1:2])
    xv = rng.normal(0.5, 2, ax)
    gv, bv = rng.uniform(0.5, 1.5, ax[1:2]), rng.uniform(0.5, 1.5, ax[1:2])
    m = ng.mean(x, out_axes=ax[1:2])
    v = ng.variance(x, out_axes=ax[1:2])
    y = gamma * ((x - m) * ng.reciprocal(ng.sqrt(v + 1e-5))) + beta
    with executor([m, v, y], x, gamma, beta) as f:
        m_g, v_g, y_g = f(xv, gv, bv)
    x64 = xv.astype(np.float64)
    m64, v64 = x64.mean(axis=(0, 2, 3)), x64.var(axis=(0, 2, 3))
    np.testing.assert_allclose(m_g, m64, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v_g, v64, rtol=1e-5, atol=1e-6)
    y64 = gv[None, :, None, None] * ((x64 - m64[None, :, None, None]) / np.sqrt(v64 + 1e-5)[None, :, None, None]) \
        + bv[None, :, None, None]
    np.testing.assert_allclose(y_g, y64, rtol=1e-5, atol=1e-5)


def test_two_group_statistics_take_one_pass_moments():
    ax = axes(N=6, C=5, H=16, W=8)
    x = ng.placeholder(ax)
    kernels = _kernels_lowered_for([ng.mean(x, out_axes=ax[1:2]), ng.variance(x, out_axes=ax[1:2])], [x])
    assert kernels[0] == "MomentsKernel" and "CopyKernel" not in kernels, kernels


def test_4d_elementwise_and_sums(backend):
    """Shapes of tests/transformer_dependent/test_kernel_generator.py:43-131."""
    for shape in [(64, 10, 28, 32), (3, 16, 16, 4), (7, 15, 19, 5), (3, 5, 7, 2)]:
        ax = ng.make_axes([ng.make_axis(n) for n in shape])
        a, b = ng.placeholder(ax), ng.placeholder(ax)
        av, bv = rng.uniform(0, 1, ax), rng.uniform(0, 1, ax)
        with executor([a + b, ng.sum(a, reduction_axes=ax[1:2]), ng.sum(a, reduction_axes=ax[3:4]),
                       ng.sum(ng.reciprocal(a + 1) + b, reduction_axes=ax[0:1])], a, b) as f:
            s, r1, r3, chain = f(av, bv)
        np.testing.assert_allclose(s, av + bv, rtol=RTOL)
        np.testing.assert_allclose(r1, av.sum(axis=1), rtol=1e-5)
        np.testing.assert_allclose(r3, av.sum(axis=3), rtol=1e-5)
        np.testing.assert_allclose(chain, (1 / (av + 1) + bv).sum(axis=0), rtol=1e-5)


def test_run_twice_bit_equal(backend):
    """Partial blocks must not leak state between calls (test_kernel_generator.py:134-160)."""
    ax = axes(H=7, W=51)
    x = ng.placeholder(ax)
    xv = rng.uniform(-1, 1, ax)
    with executor(ng.tanh(x) * 3, x) as f:
        a = f(xv).copy()
        b = f(xv)
    np.testing.assert_array_equal(a, b)


def test_log_softmax_twice_bit_equal(backend):
    """test_kernel_generator.py:43-71 (exit condition): log(softmax(y)) over the class axis of a
    16 x 10 tensor, evaluated twice with identical bits, and equal to the NumPy statement."""
    N, Y = ng.make_axis(16, name="N"), ng.make_axis(10, name="Y")
    yv = rng.uniform(-3, 3, ng.make_axes([N, Y]))
    y = ng.constant(yv, ng.make_axes([N, Y]))
    with executor(ng.log(ng.softmax(y, normalization_axes=y.axes[1]))) as f:
        a = np.array(f()).copy()
        b = np.array(f())
    np.testing.assert_array_equal(a, b)
    e = np.exp(yv - yv.max(axis=1, keepdims=True))
    np.testing.assert_allclose(a, np.log(e / e.sum(axis=1, keepdims=True)), rtol=1e-5, atol=1e-6)


def test_broadcast_add_over_a_long_trailing_axis(backend):
    """test_kernel_generator.py:174-203 (kernel cache): x[32,32] broadcast against two
    [32,32,16384] tensors."""
    X, Y, C = ng.make_axis(32, name="X"), ng.make_axis(32, name="Y"), ng.make_axis(16384, name="C")
    xv = rng.uniform(-1, 1, ng.make_axes([X, Y]))
    yv = rng.uniform(-1, 1, ng.make_axes([X, Y, C]))
    zv = rng.uniform(-1, 1, ng.make_axes([X, Y, C]))
    x, y, z = ng.constant(xv, [X, Y]), ng.constant(yv, [X, Y, C]), ng.constant(zv, [X, Y, C])
    with executor(ng.add(ng.add(x, y), z)) as f:
        np.testing.assert_allclose(f(), xv.reshape(32, 32, 1) + yv + zv, rtol=1e-6, atol=1e-6)


def test_views_reorder_slice_flatten(backend):
    C, H, N = ng.make_axis(4, name="C"), ng.make_axis(6, name="H"), ng.make_axis(5, name="N")
    x = ng.placeholder([C, H, N])
    xv = rng.uniform(-1, 1, x.axes)
    t = ng.axes_with_order(x, [N, C, H])
    s = ng.tensor_slice(x, [slice(1, 3), slice(None), 2])
    fl = ng.flatten(x, ng.make_axes([C, ng.make_axes([H, N]).flatten(force=True)]))
    with executor([t * 2, s + 1, ng.sum(fl, out_axes=[C])], x) as f:
        tv, sv, fv = f(xv)
    np.testing.assert_allclose(tv, xv.transpose(2, 0, 1) * 2, rtol=RTOL)
    np.testing.assert_allclose(sv, xv[1:3, :, 2] + 1, rtol=RTOL)
    np.testing.assert_allclose(fv, xv.reshape(4, -1).sum(axis=1), rtol=1e-5)


def test_transposed_flatten_needs_copy(backend):
    C, H = ng.make_axis(6, name="C"), ng.make_axis(10, name="H")
    x = ng.placeholder([C, H])
    xv = rng.uniform(-1, 1, x.axes)
    y = ng.flatten(ng.axes_with_order(x, [H, C]))       # not a view: a device copy is inserted
    with executor(y * 2, x) as f:
        np.testing.assert_allclose(f(xv), xv.T.reshape(-1) * 2, rtol=RTOL)


def test_assign_and_sequential_state(backend):
    """State persists across calls; sequential orders reads after writes."""
    ax = axes(H=5)
    w = ng.variable(ax, initial_value=np.arange(5, dtype=np.float32))
    x = ng.placeholder(ax)
    step = ng.sequential([ng.assign(w, w + x), w * 1.0])
    with executor(step, x) as f:
        ones = np.ones(5, dtype=np.float32)
        np.testing.assert_allclose(f(ones), np.arange(5) + 1)
        np.testing.assert_allclose(f(ones), np.arange(5) + 2)
        np.testing.assert_allclose(f(2 * ones), np.arange(5) + 4)


def test_onehot(backend):
    C, N = ng.make_axis(5, name="C"), ng.make_axis(11, name="N")
    x = ng.placeholder([N])
    xv = np.array([0, 1, 2, 3, 4, 4, 3, 2, 1, 0, 2], dtype=np.float32)
    with executor(ng.one_hot(x, axis=C), x) as f:
        np.testing.assert_array_equal(f(xv), np.eye(5, dtype=np.float32)[:, xv.astype(int)])


@pytest.mark.parametrize("lut_axis", [0, 1])
def test_lookuptable_forward(backend, lut_axis):
    """LookupTableOp fprop = the "take" template (gputransform.py:197-199) against
    ndarray.take (cpuengine.py:421-422), alone and fused into a following chain."""
    a = axes(V=50, F=24, I=37)
    V, F, I = a
    lut_axes = [V, F] if lut_axis == 0 else [F, V]
    out_axes = [I, F] if lut_axis == 0 else [F, I]
    lut = ng.placeholder(lut_axes)
    idx = ng.placeholder([I])
    looked = ng.lookuptable(lut, idx, out_axes)
    rs = np.random.RandomState(11)
    lut_np = rs.normal(0, 1, [x.length for x in lut_axes]).astype(np.float32)
    idx_np = rs.randint(0, 50, 37).astype(np.float32)
    want = lut_np.take(idx_np.astype(int), lut_axis)
    with executor([looked, ng.tanh(looked * 2.0) + 1.0, ng.sum(looked, out_axes=[F])], lut, idx) as f:
        got, chained, summed = f(lut_np, idx_np)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_allclose(chained, np.tanh(want * np.float32(2.0)) + 1.0, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(summed, want.sum(axis=lut_axis), rtol=RTOL, atol=1e-5)


def test_rng_uniform_ranges(backend):
    """tests/transformer_dependent/test_rngop.py:36-62: ranges of ng.uniform."""
    a = axes(M=5, N=8)
    t = ng.persistent_tensor(a, initial_value=10.0)
    with executor([ng.uniform(t, low=0.0, high=0.5), ng.uniform(t, low=-0.5, high=0.5)]) as f:
        pos, posneg = f()
        assert np.all(pos < 0.5) and np.all(pos >= 0.0) and not np.all(pos == 0.0)
        assert np.all(posneg < 0.5) and np.all(posneg >= -0.5) and not np.all(posneg >= 0.0)
        assert not np.array_equal(pos - 0.25, posneg * 0.5)      # two fills, two streams


def test_rng_runs_at_every_execution(backend):
    """test_rngop.py:65-79: a random fill is redone by every call of the computation."""
    a = axes(A=2, B=2)
    x = ng.variable(a, initial_value=np.array([[1, 2], [3, 4]]))
    with executor(ng.sum(ng.uniform(x), out_axes=())) as f:
        assert np.array(f()).copy() != np.array(f()).copy()


def test_rng_normal_moments(backend):
    """test_rngop.py:82-103 at a size where the moments are tight: mean, spread, and (for the
    uniform) the variance (high-low)^2/12."""
    a = axes(M=300, N=400)
    t = ng.persistent_tensor(a, initial_value=10.0)
    with executor([ng.normal(t, loc=-0.5, scale=1.0), ng.uniform(t, low=1.0, high=3.0)]) as f:
        z, u = f()
        assert abs(z.mean() + 0.5) < 0.02 and abs(z.std() - 1.0) < 0.02
        assert not np.all(z >= 0.0) and not np.all(z < 0.0)
        assert abs(np.mean(((z + 0.5)) ** 3)) < 0.05 and abs(np.mean((z + 0.5) ** 4) - 3.0) < 0.15
        assert abs(u.mean() - 2.0) < 0.01 and abs(u.var() - 4.0 / 12.0) < 0.01
        # neighbours are uncorrelated
        assert abs(np.corrcoef(u.ravel()[:-1], u.ravel()[1:])[0, 1]) < 0.02


def test_lookuptable_argument_checks():
    a = axes(V=5, F=4, I=3)
    V, F, I = a
    lut, idx = ng.placeholder([V, F]), ng.placeholder([I])
    with pytest.raises(ValueError):
        ng.lookuptable(ng.placeholder([V]), idx, [I, F])
    with pytest.raises(ValueError):
        ng.lookuptable(lut, ng.placeholder([I, F]), [I, F])
    with pytest.raises(ValueError):
        ng.lookuptable(lut, idx, [F, I])           # would transpose the table implicitly
    assert ng.lookuptable(lut, idx, [I, F]).lut_axis == 0


def test_softmax_and_simple_prune(backend):
    C, N = ng.make_axis(10, name="C"), ng.make_axis(6, name="N")
    x = ng.placeholder([C, N])
    xv = rng.uniform(-3, 3, x.axes)
    sm = ng.softmax(x, normalization_axes=ng.make_axes([C]))
    pruned = (x * 1 + 0) * -1 + ng.log(ng.exp(x))       # == 0 after SimplePrune
    with executor([sm, pruned], x) as f:
        smv, pv = f(xv)
    e = np.exp(xv - xv.max(axis=0))
    np.testing.assert_allclose(smv, e / e.sum(axis=0), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(pv, np.zeros_like(xv), atol=1e-6)


def test_computation_return_shapes_and_errors(backend):
    ax = axes(H=3)
    x, y = ng.placeholder(ax), ng.placeholder(ax)
    t = ngt.make_transformer()
    a, b = x + y, x * y
    f_seq = t.computation([a, b], x, y)
    f_set = t.computation({a, b}, x, y)
    f_one = t.computation(a, x, y)
    xv, yv = np.array([1, 2, 3], np.float32), np.array([4, 5, 6], np.float32)
    r = f_seq(xv, yv)
    assert isinstance(r, tuple) and len(r) == 2
    d = f_set(xv, yv)
    assert set(d.keys()) == {a, b}
    np.testing.assert_allclose(d[b], xv * yv)
    np.testing.assert_allclose(f_one(feed_dict={x: xv, y: yv}), xv + yv)
    with pytest.raises(ValueError):
        f_one(xv)                                # wrong argument count
    with pytest.raises(ValueError):
        t.computation(a, x, y)                   # transformer already finalized
    with pytest.raises(ValueError):
        ng.computation(a, x)                     # placeholder y not supplied
    t.close()


def test_long_chains_split_into_several_kernels(backend):
    """More ops, constants and distinct operands than one kernel spec holds: the planner has to
    cut the group, and the pieces must still compute the same values."""
    a = axes(A=33, B=70)
    xs = [ng.placeholder(a) for _ in range(14)]             # more operands than a spec's 12 slots
    vals = [rng.uniform(0.5, 1.5, a) for _ in xs]
    acc, want = xs[0], vals[0].astype(np.float64)
    for i in range(1, len(xs)):
        acc = acc * (1.0 + 0.01 * i) + xs[i]                 # a new constant each step (> 16 in all)
        want = want * (1.0 + 0.01 * i) + vals[i]
    for j in range(60):                                      # and well over 96 ops
        acc = ng.tanh(acc * 0.5) + (0.25 + 0.001 * j)
        want = np.tanh(want * 0.5) + (0.25 + 0.001 * j)
    with executor(acc, *xs) as f:
        np.testing.assert_allclose(f(*vals), want, rtol=2e-5, atol=2e-6)


def test_more_than_four_reductions_of_one_tensor(backend):
    a = axes(R=50, N=40)
    x = ng.placeholder(a)
    xv = rng.uniform(0.5, 1.5, a)
    outs = [ng.sum(x, out_axes=[a[1]]), ng.max(x, out_axes=[a[1]]), ng.min(x, out_axes=[a[1]]),
            ng.prod(x * 0.9, out_axes=[a[1]]), ng.argmax(x, out_axes=[a[1]]), ng.argmin(x, out_axes=[a[1]]),
            ng.sum(x * x, out_axes=[a[1]])]
    with executor(outs, x) as f:
        s, mx, mn, pr, am, an, ss = f(xv)
    np.testing.assert_allclose(s, xv.sum(0), rtol=1e-5)
    np.testing.assert_array_equal(mx, xv.max(0))
    np.testing.assert_array_equal(mn, xv.min(0))
    np.testing.assert_allclose(pr, (xv * np.float32(0.9)).prod(0), rtol=1e-4)
    np.testing.assert_array_equal(am, xv.argmax(0))
    np.testing.assert_array_equal(an, xv.argmin(0))
    np.testing.assert_allclose(ss, (xv * xv).sum(0), rtol=1e-5)


# ---- cross entropies (reference tests/transformer_dependent/test_execution.py:584-598, 786-813, 863-897)

def _np_softmax(x, axis):
    e = np.exp(x - x.max(axis=axis, keepdims=True))
    return e / e.sum(axis=axis, keepdims=True)


def test_cross_entropy_binary_logistic_shortcut(backend):
    C, N = ng.make_axis(3, name="C"), ng.make_axis(8, name="N")
    p_u, p_v = ng.placeholder([C, N]), ng.placeholder([C, N])
    u = rng.uniform(-3.0, 3.0, p_u.axes)
    v = _np_softmax(rng.uniform(-3.0, 3.0, p_u.axes), 0).astype(np.float32)
    y = 1.0 / (1.0 + np.exp(-u.astype(np.float64)))
    want = -(v * np.log(y) + (1.0 - v) * np.log(1.0 - y))
    short = ng.cross_entropy_binary_inner(ng.sigmoid(p_u), p_v)
    plain = ng.cross_entropy_binary_inner(ng.sigmoid(p_u), p_v, enable_sig_opt=False)
    total = ng.cross_entropy_binary(ng.sigmoid(p_u), p_v, usebits=True)
    with executor([short, plain, total], p_u, p_v) as f:
        s, p, tot = f(u, v)
    np.testing.assert_allclose(s, want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(p, want, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(tot, want.sum(axis=0) / np.log(2.0), rtol=1e-5)


@pytest.mark.parametrize("recurrent", [False, True])
def test_cross_entropy_softmax(backend, recurrent):
    C, N = ng.make_axis(3, name="C"), ng.make_axis(8, name="N")
    ax = [C, ng.make_axis(4, name="REC"), N] if recurrent else [C, N]
    p_x, p_t = ng.placeholder(ax), ng.placeholder(ax)
    x = rng.uniform(0, 1, p_x.axes)
    t = _np_softmax(rng.uniform(0, 1, p_t.axes), 0).astype(np.float32)
    want = -(np.log(_np_softmax(x.astype(np.float64), 0)) * t).sum(axis=0)
    short = ng.cross_entropy_multi(ng.softmax(p_x), p_t)
    plain = ng.cross_entropy_multi(ng.softmax(p_x), p_t, enable_softmax_opt=False)
    with executor([short, plain], p_x, p_t) as f:
        s, p = f(x, t)
    assert s.shape == want.shape
    np.testing.assert_allclose(s, want, rtol=1e-5)
    np.testing.assert_allclose(p, want, rtol=1e-5)


def test_cross_entropy_softmax_large_input(backend):
    C, N = ng.make_axis(3, name="C"), ng.make_axis(8, name="N")
    p_x, p_t = ng.placeholder([C, N]), ng.placeholder([C, N])
    r = np.random.RandomState(3)
    x = (np.eye(3)[r.choice(3, 8)].T * rng.uniform(-10, 10, p_x.axes) * 25).astype(np.float32)
    t = np.eye(3)[r.choice(3, 8)].T.astype(np.float32)
    x64 = x.astype(np.float64)
    logsm = x64 - x64.max(axis=0) - np.log(np.exp(x64 - x64.max(axis=0)).sum(axis=0))
    want = np.minimum(-(logsm * t).sum(axis=0), 50.0)
    with executor(ng.cross_entropy_multi(ng.softmax(p_x), p_t), p_x, p_t) as f:
        np.testing.assert_allclose(f(x, t), want, atol=1e-7, rtol=1e-4)


def test_cross_entropy_axis_checks_and_order(backend):
    C, N = ng.make_axis(5, name="C"), ng.make_axis(8, name="N")
    y = ng.placeholder([C, N])
    with pytest.raises(ng.UnmatchedAxesError):
        ng.cross_entropy_multi(y, ng.placeholder([ng.make_axis(5), N]))
    with pytest.raises(ng.UnmatchedAxesError):
        ng.cross_entropy_binary_inner(y, ng.placeholder([ng.make_axis(5), N]))
    t1, t2 = ng.placeholder([C, N]), ng.placeholder([N, C])
    yv = rng.uniform(0, 1, y.axes)
    t1v = np.eye(8, dtype=np.float32)[:5, :]
    with executor([ng.cross_entropy_multi(ng.softmax(y), t1),
                   ng.cross_entropy_multi(ng.softmax(y), t2)], y, t1, t2) as f:
        a, b = f(yv, t1v, np.ascontiguousarray(t1v.T))
    np.testing.assert_allclose(a, b, rtol=1e-6)


# ---- small forward cases (reference test_execution.py:990-1065, 1122-1150, 1208-1216)

def test_clip(backend):
    a = axes(W=4, H=5)
    p_x = ng.placeholder(a)
    x = (2 * rng.uniform(0, 1, a) - 1) * 20
    with executor(ng.minimum(ng.maximum(p_x, -10), 10), p_x) as f:
        np.testing.assert_array_equal(f(x), np.clip(x, -10, 10))


def test_elementwise_fp16_in_and_out(backend):
    a = axes(A=2, B=2)
    h1 = ng.constant(np.array([[1.0, 2.0], [4.0, 12.0]], dtype="float16"), a, dtype=np.dtype(np.float16))
    h2 = ng.constant(np.array([[1.0, 2.0], [6.0, 12.0]], dtype="float16"), a, dtype=np.dtype(np.float16))
    f1 = ng.constant(np.array([[1.0, 2.0], [4.0, 12.0]], dtype="float32"), a)
    f2 = ng.constant(np.array([[1.0, 2.0], [6.0, 12.0]], dtype="float32"), a)
    with executor([ng.multiply(h1, h2), ng.multiply(f1, f2, dtype=np.dtype(np.float16))]) as f:
        r_in, r_out = f()
    np.testing.assert_array_equal(r_in, [[1.0, 4.0], [24.0, 144.0]])
    np.testing.assert_array_equal(r_out, [[1.0, 4.0], [24.0, 144.0]])
    assert r_out.dtype == np.float16


def test_fill_slice(backend):
    a = axes(A=2, B=8)
    x = ng.placeholder(a)
    b = ng.sequential([ng.fill(x[:, 1], 0), ng.value_of(x)])
    with executor(b, x) as f:
        got = f(np.array([[1, 2, 3, 4, 5, 6, 7, 8], [8, 7, 6, 5, 4, 3, 2, 1]], dtype=np.float32))
    np.testing.assert_array_equal(got, [[1, 0, 3, 4, 5, 6, 7, 8], [8, 0, 6, 5, 4, 3, 2, 1]])


def test_empty_transformer_initializes(backend):
    t = ngt.make_transformer()
    t.initialize()
    t.close()


def test_variance_sqrt_inverse_forward(backend):
    C, N = ng.make_axis(7, name="C"), ng.make_axis(16, name="N")
    x, tg = ng.placeholder([C, N]), ng.placeholder([C, N])
    stat = ng.reciprocal(ng.sqrt(ng.variance(x, reduction_axes=x.axes.batch_axes()) + 1e-3))
    err = ng.sum(stat - tg, out_axes=())
    xv, tv = rng.uniform(-1, 1, x.axes), rng.uniform(-1, 1, x.axes)
    with executor(err, x, tg) as f:
        got = f(xv, tv)
    want = np.sum(1.0 / np.sqrt(np.var(xv.astype(np.float64), axis=1, keepdims=True) + 1e-3) - tv)
    np.testing.assert_allclose(got, want, atol=1e-4, rtol=1e-4)


def test_moving_32_bit_integers_keeps_every_bit(backend):
    """Kernel registers are fp32 (exact up to 2**24); a kernel that only moves int32 / uint32
    values must not round them all the same."""
    ax = axes(H=6)
    for dtype, values in ((np.int32, [0, 16777217, -16777219, 2 ** 31 - 1, -2 ** 31, 123456789]),
                          (np.uint32, [0, 16777217, 2 ** 32 - 1, 2 ** 31 + 1, 4000000001, 7])):
        v = ng.variable(ax, dtype=dtype, initial_value=np.zeros(6, dtype=dtype))
        x = ng.placeholder(ax, dtype=dtype)
        with executor(ng.sequential([ng.assign(v, x), v]), x) as f:
            got = np.array(f(np.array(values, dtype=dtype)))
        assert got.dtype == dtype
        np.testing.assert_array_equal(got, np.array(values, dtype=dtype))


def test_integer_operands_meet_in_integer_arithmetic(backend):
    """An op all of whose operands are int32 (or all uint32) computes as NumPy's integer loops
    and C's integer operators do -- exactly, wrapping at 2**32 -- and only its result is
    converted to the op's own type (float_ew2.py:615-641: `int` registers; cputransform.py hands
    the integer arrays to the ufuncs as they are).  Where an integer meets a float the integer
    is converted first."""
    ax = axes(H=8)
    a = np.array([16777217, 2 ** 31 - 1, -2 ** 31, 123456789, -16777219, 5, -7, 0], dtype=np.int32)
    b = np.array([16777217, 1, -1, 987654321, 3, -5, 7, 0], dtype=np.int32)
    x, y = ng.placeholder(ax, dtype=np.int32), ng.placeholder(ax, dtype=np.int32)
    results = [x + y, x - y, x * y, ng.maximum(x, y), ng.minimum(x, y), -x, ng.absolute(x),
               ng.equal(x, y), ng.less(x, y), ng.greater_equal(x, y),
               ng.add(x, y, dtype=np.int32),                                   # stays an integer
               (x + y) * 0.5,                                                   # converted, then float
               ng.multiply(ng.add(x, y, dtype=np.int32), ng.subtract(x, y, dtype=np.int32))]
    with np.errstate(over="ignore"):
        s, d = a + b, a - b
        want = [s.astype(np.float32), d.astype(np.float32), (a * b).astype(np.float32),
                np.maximum(a, b).astype(np.float32), np.minimum(a, b).astype(np.float32),
                (-a).astype(np.float32), np.abs(a).astype(np.float32),
                (a == b).astype(np.float32), (a < b).astype(np.float32), (a >= b).astype(np.float32),
                s, s.astype(np.float32) * np.float32(0.5), (s * d).astype(np.float32)]
    with executor(results, x, y) as f:
        got = f(a, b)
    for i, (g, w) in enumerate(zip(got, want)):
        g = np.array(g)
        assert g.dtype == w.dtype, (i, g.dtype, w.dtype)
        np.testing.assert_array_equal(g, w, err_msg="result %d" % i)
    # unsigned: wraps modulo 2**32, compares as unsigned
    ua = np.array([2 ** 32 - 1, 2 ** 31 + 5, 16777217, 7, 0, 4000000000, 1, 2 ** 31], dtype=np.uint32)
    ub = np.array([1, 2 ** 31 + 5, 16777217, 9, 0, 300000000, 2 ** 32 - 1, 2 ** 31 - 1], dtype=np.uint32)
    u, v = ng.placeholder(ax, dtype=np.uint32), ng.placeholder(ax, dtype=np.uint32)
    with np.errstate(over="ignore"):
        want = [(ua + ub).astype(np.float32), (ua * ub).astype(np.float32), np.maximum(ua, ub).astype(np.float32),
                (ua < ub).astype(np.float32), (ua >= ub).astype(np.float32), ua + ub]
    with executor([u + v, u * v, ng.maximum(u, v), ng.less(u, v), ng.greater_equal(u, v),
                   ng.add(u, v, dtype=np.uint32)], u, v) as f:
        got = f(ua, ub)
    for i, (g, w) in enumerate(zip(got, want)):
        g = np.array(g)
        assert g.dtype == w.dtype, (i, g.dtype, w.dtype)
        np.testing.assert_array_equal(g, w, err_msg="unsigned result %d" % i)


def test_integer_tensor_moved_and_written_through_a_conversion_in_one_kernel(backend):
    """The same int32 tensor read as integers and overwritten with a float result in one kernel:
    one binding cannot serve both ways, so such a kernel keeps floats throughout (values below
    2**24 are exact either way)."""
    ax = axes(H=6)
    v = ng.variable(ax, dtype=np.int32, initial_value=np.array([1, -2, 3, 70000, -5, 6], dtype=np.int32))
    x = ng.placeholder(ax, dtype=np.int32)
    step = ng.sequential([ng.assign(v, (v + x) * 0.5), v])
    with executor(step, x) as f:
        got = np.array(f(np.array([3, 4, -9, 10, 5, 1], dtype=np.int32)))
    np.testing.assert_array_equal(got, np.array([2, 1, -3, 35005, 0, 3], dtype=np.int32))


def test_multiply_uint32_scalar(backend):
    x = ng.placeholder((), dtype=np.uint32)
    with executor(0.5 * x * 0.5, x) as f:
        assert f(1) == 0.25
