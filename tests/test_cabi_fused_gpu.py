"""Parity of the fused kernels, driven through the C ABI with hand-built specs.

Each case builds an ngh_fused_spec the way the transformer's lowering does,
launches it with ngh_launch_fused and compares with the CPU oracle
(oracle/configs.py, oracle/numpy_ops.py) on the same seeded inputs.
Tolerance: fp32 rtol 1e-5 / atol 1e-6.
"""
import numpy as np
import pytest

from oracle import configs, numpy_ops
from ngraph_hip.runtime import FusedSpecBuilder, NGH_F32, NGH_I32
from ngraph_hip.runtime.hiplib import (FLOAT_UNARY_OPS, FLOAT_BINARY_OPS, INTEGER_UNARY_OPS,
                                       INTEGER_BINARY_OPS)
from conftest import default_kernel_choice

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6
f32 = np.float32


def contiguous_strides(shape):
    strides, acc = [], 1
    for s in reversed(shape):
        strides.insert(0, acc)
        acc *= s
    return strides


def c1_spec(rt, x_d, a_d, b_d, y_d, shape):
    st = contiguous_strides(shape)
    z = [0] * len(shape)
    sb = FusedSpecBuilder(shape)
    tx, ta, tb, ty = (sb.tensor(x_d.ptr, st), sb.tensor(a_d.ptr, z), sb.tensor(b_d.ptr, z),
                      sb.tensor(y_d.ptr, st))
    x = sb.load(tx)
    a = sb.load(ta)
    b = sb.load(tb)
    t = sb.binary("mul", a, x)
    t = sb.binary("add", t, b)
    t = sb.unary("tanh", t)
    u = sb.unary("neg", x)
    u = sb.unary("exp", u)
    one = sb.constant(1.0)
    u = sb.binary("add", u, one)
    u = sb.unary("rcp", u)
    y = sb.binary("mul", t, u)
    sb.store(ty, y)
    return sb.build()


@pytest.mark.parametrize("shape", [(1024, 1024), (7, 33), (1, 5), (3, 4, 5), (1000003,)])
def test_c1_tanh_sigmoid_chain(hip_runtime, shape):
    rt = hip_runtime
    x, a, b = configs.c1_inputs(shape, seed=0)
    want = configs.c1_cpu(x, a, b)
    x_d, a_d, b_d = rt.array(x), rt.array(np.array([a])), rt.array(np.array([b]))
    y_d = rt.empty(shape)
    spec = c1_spec(rt, x_d, a_d, b_d, y_d, shape)
    rt.launch_fused(spec)
    got = y_d.get()
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    for d in (x_d, a_d, b_d, y_d):
        d.free()


def bn_specs(rt, x_d, g_d, b_d, y_d, mean_d, var_d, C, R, eps):
    """Reference-faithful staging: sum -> mean, sum((x-mean)^2) -> var, normalise.

    View is [R, C] with the reduced axis first (gputransform.py:117-122);
    memory is [C, R] so strides are (1, R).
    """
    xs, cs = [1, R], [0, 1]
    sb = FusedSpecBuilder([R, C])
    tx = sb.tensor(x_d.ptr, xs)
    tmean = sb.tensor(mean_d.ptr, cs)
    x = sb.load(tx)
    sb.reduce("sum", x, tmean)
    s1 = sb.build()

    sb = FusedSpecBuilder([C])
    tmean = sb.tensor(mean_d.ptr, [1])
    m = sb.load(tmean)
    n = sb.constant(R)
    m = sb.binary("div", m, n)
    sb.store(tmean, m)
    s2 = sb.build()

    sb = FusedSpecBuilder([R, C])
    tx = sb.tensor(x_d.ptr, xs)
    tmean = sb.tensor(mean_d.ptr, cs)
    tvar = sb.tensor(var_d.ptr, cs)
    x = sb.load(tx)
    m = sb.load(tmean)
    d = sb.binary("sub", x, m)
    d = sb.unary("sqr", d)
    sb.reduce("sum", d, tvar)
    s3 = sb.build()

    sb = FusedSpecBuilder([C])
    tvar = sb.tensor(var_d.ptr, [1])
    v = sb.load(tvar)
    n = sb.constant(R)
    v = sb.binary("div", v, n)
    sb.store(tvar, v)
    s4 = sb.build()

    sb = FusedSpecBuilder([R, C])
    tx = sb.tensor(x_d.ptr, xs)
    tmean = sb.tensor(mean_d.ptr, cs)
    tvar = sb.tensor(var_d.ptr, cs)
    tg = sb.tensor(g_d.ptr, cs)
    tb = sb.tensor(b_d.ptr, cs)
    ty = sb.tensor(y_d.ptr, xs)
    x = sb.load(tx)
    m = sb.load(tmean)
    v = sb.load(tvar)
    d = sb.binary("sub", x, m)
    e = sb.constant(eps)
    r = sb.binary("add", v, e)
    r = sb.unary("sqrt", r)
    r = sb.unary("rcp", r)
    d = sb.binary("mul", d, r)
    g = sb.load(tg)
    d = sb.binary("mul", g, d)
    bb = sb.load(tb)
    d = sb.binary("add", d, bb)
    sb.store(ty, d)
    s5 = sb.build()
    return [s1, s2, s3, s4, s5]


@pytest.mark.parametrize("C,R", [(16, 4096), (3, 1000), (256, 56 * 56), (5, 17)])
def test_c2_batchnorm_staged(hip_runtime, C, R):
    rt = hip_runtime
    x, gamma, beta = configs.c2_inputs(C, R, seed=1)
    y_w, mean_w, var_w = configs.c2_cpu(x, gamma, beta)
    x_d, g_d, b_d = rt.array(x), rt.array(gamma), rt.array(beta)
    y_d, mean_d, var_d = rt.empty((C, R)), rt.empty((C,)), rt.empty((C,))
    for spec in bn_specs(rt, x_d, g_d, b_d, y_d, mean_d, var_d, C, R, 1e-5):
        rt.launch_fused(spec)
    np.testing.assert_allclose(mean_d.get(), mean_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var_d.get(), var_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y_d.get(), y_w, rtol=RTOL, atol=1e-5)
    for d in (x_d, g_d, b_d, y_d, mean_d, var_d):
        d.free()


def adam_spec(rt, p_d, g_d, m_d, v_d, n, ell, beta1, beta2, eps):
    sb = FusedSpecBuilder([n])
    tp, tg, tm, tv = (sb.tensor(d.ptr, [1]) for d in (p_d, g_d, m_d, v_d))
    b1, b2 = f32(beta1), f32(beta2)
    g = sb.load(tg)
    m = sb.load(tm)
    a = sb.binary("mul", m, sb.constant(b1))
    b = sb.binary("mul", sb.constant(f32(1) - b1), g)
    m = sb.binary("add", a, b)
    sb.store(tm, m)
    v = sb.load(tv)
    a = sb.binary("mul", v, sb.constant(b2))
    b = sb.binary("mul", sb.constant(f32(1) - b2), g)
    b = sb.binary("mul", b, g)
    v = sb.binary("add", a, b)
    sb.store(tv, v)
    a = sb.binary("mul", sb.constant(ell), m)
    b = sb.unary("sqrt", v)
    b = sb.binary("add", b, sb.constant(eps))
    a = sb.binary("div", a, b)
    p = sb.load(tp)
    p = sb.binary("sub", p, a)
    sb.store(tp, p)
    return sb.build()


@pytest.mark.parametrize("n", [1 << 20, 1000003, 13])
def test_c3_adam_in_place(hip_runtime, n):
    rt = hip_runtime
    p, g, m, v = configs.c3_inputs(n, seed=2)
    p_d, g_d, m_d, v_d = rt.array(p), rt.array(g), rt.array(m), rt.array(v)
    for t in (1, 2):
        configs.c3_cpu(p, g, m, v, t)
        rt.launch_fused(adam_spec(rt, p_d, g_d, m_d, v_d, n, configs.adam_ell(t), 0.9, 0.999, 1e-8))
    np.testing.assert_allclose(m_d.get(), m, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v_d.get(), v, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(p_d.get(), p, rtol=RTOL, atol=ATOL)
    for d in (p_d, g_d, m_d, v_d):
        d.free()


def lstm_specs(rt, gates_d, cprev_d, c_d, h_d, db_d, H, N):
    # logical [H, N] views of the transposed storage: strides (1, 4H) / (1, H)
    gs, cs, os_ = [1, 4 * H], [1, H], [N, 1]
    sb = FusedSpecBuilder([H, N])
    itemsize = 4
    tg = [sb.tensor(gates_d.ptr + k * H * itemsize, gs) for k in range(4)]
    tc_prev = sb.tensor(cprev_d.ptr, cs)
    tc = sb.tensor(c_d.ptr, os_)
    th = sb.tensor(h_d.ptr, os_)

    def sigmoid(r):
        r = sb.unary("neg", r)
        r = sb.unary("exp", r)
        r = sb.binary("add", r, sb.constant(1.0))
        return sb.unary("rcp", r)

    i = sigmoid(sb.load(tg[0]))
    f = sigmoid(sb.load(tg[1]))
    o = sigmoid(sb.load(tg[2]))
    g = sb.unary("tanh", sb.load(tg[3]))
    c = sb.binary("mul", f, sb.load(tc_prev))
    ig = sb.binary("mul", i, g)
    c = sb.binary("add", c, ig)
    sb.store(tc, c)
    tc_act = sb.unary("tanh", c)
    h = sb.binary("mul", o, tc_act)
    sb.store(th, h)
    s1 = sb.build()

    # db = sum over N of gates: view [N, 4H] with the reduced axis first
    sb = FusedSpecBuilder([N, 4 * H])
    tg_all = sb.tensor(gates_d.ptr, [4 * H, 1])
    tdb = sb.tensor(db_d.ptr, [0, 1])
    sb.reduce("sum", sb.load(tg_all), tdb)
    s2 = sb.build()
    return [s1, s2]


@pytest.mark.parametrize("H,N", [(1024, 64), (96, 7), (64, 64)])
def test_c4_lstm_cell_transposed(hip_runtime, H, N):
    rt = hip_runtime
    gates, cprev = configs.c4_inputs(H, N, seed=3)
    c_w, h_w, db_w = configs.c4_cpu(gates, cprev)
    gates_d, cprev_d = rt.array(gates), rt.array(cprev)
    c_d, h_d, db_d = rt.empty((H, N)), rt.empty((H, N)), rt.empty((4 * H,))
    for spec in lstm_specs(rt, gates_d, cprev_d, c_d, h_d, db_d, H, N):
        rt.launch_fused(spec)
    np.testing.assert_allclose(c_d.get(), c_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(h_d.get(), h_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(db_d.get(), db_w, rtol=RTOL, atol=1e-5)
    for d in (gates_d, cprev_d, c_d, h_d, db_d):
        d.free()


@pytest.mark.parametrize("H,N", [(1024, 64), (96, 7), (64, 64)])
def test_c4_cell_and_bias_gradient_as_one_launch(hip_runtime, H, N):
    """The LSTM cell and the column sum for its bias gradient depend on nothing of each other:
    ngh_launch_fused_pair takes them in one call, whichever spec comes first, and gives the
    results of the two launches.  (ONE launch needs the library's own pair of programs, which
    the cell as the transformer lowers it matches -- tests/test_configs.py::test_c4_graph
    checks that path -- and this hand-written cell does not: the call reports which it was.)"""
    rt = hip_runtime
    gates, cprev = configs.c4_inputs(H, N, seed=5)
    c_w, h_w, db_w = configs.c4_cpu(gates, cprev)
    gates_d, cprev_d = rt.array(gates), rt.array(cprev)
    for swap in (False, True):
        c_d, h_d, db_d = rt.empty((H, N)), rt.empty((H, N)), rt.empty((4 * H,))
        for d in (c_d, h_d, db_d):
            d.set(np.full(d.shape, np.nan, f32))
        cell, bias = lstm_specs(rt, gates_d, cprev_d, c_d, h_d, db_d, H, N)
        paired = rt.describe_fused(cell, 0) == "special:lstm_cell_k0" and \
            rt.describe_fused(bias, 0) == "special:sum_across_small_k0"
        one = rt.launch_fused_pair(bias, cell) if swap else rt.launch_fused_pair(cell, bias)
        assert one == paired
        np.testing.assert_allclose(c_d.get(), c_w, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(h_d.get(), h_w, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(db_d.get(), db_w, rtol=RTOL, atol=1e-5)
        for d in (c_d, h_d, db_d):
            d.free()
    gates_d.free()
    cprev_d.free()


def test_a_pair_the_library_has_no_kernel_for_is_two_launches(hip_runtime):
    rt = hip_runtime
    n = 4099
    x = np.random.RandomState(2).normal(0, 1, n).astype(f32)
    x_d, y_d, z_d = rt.array(x), rt.empty((n,)), rt.empty((n,))
    specs = []
    for out, name in ((y_d, "tanh"), (z_d, "exp")):
        sb = FusedSpecBuilder([n])
        sb.store(sb.tensor(out.ptr, [1]), sb.unary(name, sb.load(sb.tensor(x_d.ptr, [1]))))
        specs.append(sb.build())
    assert not rt.launch_fused_pair(specs[0], specs[1])
    np.testing.assert_allclose(y_d.get(), numpy_ops.unary("tanh", x), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(z_d.get(), numpy_ops.unary("exp", x), rtol=RTOL, atol=ATOL)
    for d in (x_d, y_d, z_d):
        d.free()


@pytest.mark.parametrize("name", FLOAT_UNARY_OPS)
def test_every_unary_op(hip_runtime, name):
    rt = hip_runtime
    rs = np.random.RandomState(11)
    x = rs.normal(0, 2, 4099).astype(f32)
    if name in ("sqrt", "log", "log2", "safelog"):
        x = np.abs(x) + f32(1e-3)
        if name == "safelog":
            x[::7] = 0
            x[1::7] = -1
    x[:3] = [0.0, 1.0, -1.0] if name not in ("sqrt", "log", "log2") else [1.0, 2.0, 0.5]
    want = numpy_ops.unary(name, x)
    x_d, y_d = rt.array(x), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.unary(name, sb.load(tx)))
    rt.launch_fused(sb.build())
    got = y_d.get()
    # transcendental results may differ from NumPy's by a couple of ulp
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
    x_d.free()
    y_d.free()


def _ulps(got, want):
    """Distance between two float32 arrays in units of the float32 spacing at `want`."""
    with np.errstate(all="ignore"):
        spacing = np.spacing(np.abs(want).astype(f32))
        d = np.abs(got.astype(np.float64) - want.astype(np.float64)) / spacing
    d[(got == want) | (np.isnan(got) & np.isnan(want))] = 0
    return d


_TRANSCENDENTAL_RANGES = {
    # name: (float64 function, sampler of n float32 arguments)
    "exp": (np.exp, lambda rs, n: rs.uniform(-104, 89, n)),
    "exp2": (np.exp2, lambda rs, n: rs.uniform(-150, 128, n)),
    "log": (np.log, lambda rs, n: np.exp(rs.uniform(np.log(1e-45), np.log(3e38), n))),
    "log2": (np.log2, lambda rs, n: np.exp(rs.uniform(np.log(1e-45), np.log(3e38), n))),
    "tanh": (np.tanh, lambda rs, n: np.concatenate([rs.uniform(-12, 12, n // 2), rs.normal(0, 1e-3, n - n // 2)])),
    "sin": (np.sin, lambda rs, n: np.concatenate([rs.uniform(-100, 100, n // 2), rs.uniform(-1e6, 1e6, n - n // 2)])),
    "cos": (np.cos, lambda rs, n: np.concatenate([rs.uniform(-100, 100, n // 2), rs.uniform(-1e6, 1e6, n - n // 2)])),
    "sqrt": (np.sqrt, lambda rs, n: np.exp(rs.uniform(np.log(1e-45), np.log(3e38), n))),
    "rcp": (lambda v: 1.0 / v, lambda rs, n: np.exp(rs.uniform(np.log(1e-38), np.log(3e38), n)) * rs.choice([-1, 1], n)),
}


@pytest.mark.parametrize("name", sorted(_TRANSCENDENTAL_RANGES))
def test_transcendental_ops_within_2_ulp(hip_runtime, name):
    """A million arguments over each function's whole float32 range, denormal results included:
    the kernel's result is within 2 units in the last place of the correctly rounded one
    (float64 NumPy, rounded), and within 4 of the oracle's float32 NumPy result, which is itself
    up to 3 away from the correctly rounded value (exp2, log) on the build machine."""
    rt = hip_runtime
    truth_fn, sample = _TRANSCENDENTAL_RANGES[name]
    x = sample(np.random.RandomState(5), 1 << 20).astype(f32)
    with np.errstate(all="ignore"):
        truth = truth_fn(x.astype(np.float64)).astype(f32)
    want = numpy_ops.unary(name, x)
    x_d, y_d = rt.array(x), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.unary(name, sb.load(tx)))
    rt.launch_fused(sb.build())
    got = y_d.get()
    x_d.free()
    y_d.free()
    d_truth, d_oracle = _ulps(got, truth), _ulps(got, want)
    assert np.isfinite(d_truth).all() and np.isfinite(d_oracle).all()      # same infinities, same NaNs
    worst = int(np.argmax(d_truth))
    assert d_truth.max() <= 2, (name, x[worst], got[worst], truth[worst])
    worst = int(np.argmax(d_oracle))
    assert d_oracle.max() <= 4, (name, x[worst], got[worst], want[worst])


def test_sigmoid_and_pow_within_ulps_of_the_oracle(hip_runtime):
    """sig is the composite 1 / (1 + exp(-x)) on both sides (op_graph.py:4183-4197): the kernel's
    exp is within 1 ulp of exact and NumPy's within 2, which the division carries into at most 4
    ulp between the two results; pow stays within 2."""
    rt = hip_runtime
    rs = np.random.RandomState(6)
    n = 1 << 20
    x = rs.uniform(-87, 87, n).astype(f32)
    want = numpy_ops.unary("sig", x)
    x_d, y_d = rt.array(x), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.unary("sig", sb.load(tx)))
    rt.launch_fused(sb.build())
    assert _ulps(y_d.get(), want).max() <= 4
    base = np.exp(rs.uniform(np.log(1e-3), np.log(1e3), n)).astype(f32)
    expo = rs.uniform(-8, 8, n).astype(f32)
    want = numpy_ops.binary("pow", base, expo)
    b_d, e_d = rt.array(base), rt.array(expo)
    sb = FusedSpecBuilder(x.shape)
    tb, te, ty = sb.tensor(b_d.ptr, [1]), sb.tensor(e_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.binary("pow", sb.load(tb), sb.load(te)))
    rt.launch_fused(sb.build())
    assert _ulps(y_d.get(), want).max() <= 2
    for d in (x_d, y_d, b_d, e_d):
        d.free()


@pytest.mark.parametrize("name", FLOAT_BINARY_OPS)
def test_every_binary_op(hip_runtime, name):
    rt = hip_runtime
    rs = np.random.RandomState(12)
    x = rs.normal(0, 3, (37, 129)).astype(f32)
    y = rs.normal(0, 3, (37, 129)).astype(f32)
    if name in ("eq", "ne", "le", "ge"):
        y[::3] = x[::3]
    if name in ("int_div", "mod"):
        x = np.round(x * 3).astype(f32)
        y = np.round(y).astype(f32)
        y[y == 0] = 2
    if name == "pow":
        x = np.abs(x) + f32(0.1)
    want = numpy_ops.binary(name, x, y)
    x_d, y_d, z_d = rt.array(x), rt.array(y), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    st = contiguous_strides(x.shape)
    tx, ty, tz = sb.tensor(x_d.ptr, st), sb.tensor(y_d.ptr, st), sb.tensor(z_d.ptr, st)
    sb.store(tz, sb.binary(name, sb.load(tx), sb.load(ty)))
    rt.launch_fused(sb.build())
    np.testing.assert_allclose(z_d.get(), want, rtol=RTOL, atol=ATOL)
    for d in (x_d, y_d, z_d):
        d.free()


_SPECIAL = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 3.0, -3.0, 2.5, -2.5, 1e-38, -1e-38, 1e-45, 3e38,
                     -3e38, 88.0, -88.0, 104.0, -104.0, 1e6, np.inf, -np.inf, np.nan], dtype=f32)


def _assert_same_special(got, want, what, zero_sign=True):
    """NaN where the oracle has NaN, the same infinities, the same sign of zero; finite values to
    the tolerance of the ordinary tests."""
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want), err_msg=what + ": NaN pattern")
    ok = ~np.isnan(want)
    inf = ok & np.isinf(want)
    np.testing.assert_array_equal(got[inf], want[inf], err_msg=what + ": infinities")
    zero = ok & (want == 0)
    np.testing.assert_array_equal(got[zero], want[zero], err_msg=what + ": zeros")
    if zero_sign:
        np.testing.assert_array_equal(np.signbit(got[zero]), np.signbit(want[zero]), err_msg=what + ": sign of zero")
    fin = ok & ~inf & ~zero
    np.testing.assert_allclose(got[fin], want[fin], rtol=RTOL, atol=0, err_msg=what)


@pytest.mark.parametrize("name", FLOAT_UNARY_OPS)
def test_unary_ops_on_special_values(hip_runtime, name):
    """Zeros of both signs, denormals, values that overflow exp, infinities and NaN go through
    every unary op like through the oracle's NumPy call (cputransform.py:512-761)."""
    rt = hip_runtime
    x = np.tile(_SPECIAL, 11)[:256 + 7]                   # a vector body and a scalar tail
    want = numpy_ops.unary(name, x)
    x_d, y_d = rt.array(x), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.unary(name, sb.load(tx)))
    rt.launch_fused(sb.build())
    got = y_d.get()
    x_d.free()
    y_d.free()
    _assert_same_special(got, want, name)


@pytest.mark.parametrize("name", FLOAT_BINARY_OPS)
def test_binary_ops_on_special_values(hip_runtime, name):
    """Every pair of the special values through every binary op: division and remainder by zero,
    NaN in comparisons, minimum / maximum with NaN, powers of zero and of negative numbers."""
    rt = hip_runtime
    x, y = (a.ravel().copy() for a in np.meshgrid(_SPECIAL, _SPECIAL, indexing="ij"))
    want = numpy_ops.binary(name, x, y)
    x_d, y_d, z_d = rt.array(x), rt.array(y), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty, tz = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1]), sb.tensor(z_d.ptr, [1])
    sb.store(tz, sb.binary(name, sb.load(tx), sb.load(ty)))
    rt.launch_fused(sb.build())
    got = z_d.get()
    for d in (x_d, y_d, z_d):
        d.free()
    # maximum(+0, -0): NumPy's vector loop returns the second operand and its scalar loop (the
    # last few elements of an array) the first, so the sign of that zero is not compared
    _assert_same_special(got, want, name, zero_sign=name not in ("minimum", "maximum"))


def _integer_patterns(seed, n):
    """32-bit patterns over the whole range with the edges of both integer types in front."""
    rs = np.random.RandomState(seed)
    x = rs.randint(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32)
    edges = np.array([0, 1, 2, 0x7fffffff, 0x80000000, 0x80000001, 0xffffffff, 0xfffffffe, 1 << 24, (1 << 24) + 1,
                      0x00ffffff, 0x7f800000, 0xff800000, 0x7fc00000], dtype=np.uint32)   # incl. the bits of inf / NaN
    x[:len(edges)] = edges
    return x


@pytest.mark.parametrize("name", INTEGER_UNARY_OPS)
def test_every_integer_unary_op(hip_runtime, name):
    """The integer ops read a register's bits as int32 / uint32: compared bit for bit with
    NumPy's integer loops over the whole 32-bit range (tensors bound as fp32 move their bits)."""
    rt = hip_runtime
    x = _integer_patterns(21, 4099)
    want = numpy_ops.integer_unary(name, x)
    x_d, y_d = rt.array(x.view(f32)), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.unary(name, sb.load(tx)))
    rt.launch_fused(sb.build())
    got = y_d.get()
    x_d.free()
    y_d.free()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("name", INTEGER_BINARY_OPS)
def test_every_integer_binary_op(hip_runtime, name):
    rt = hip_runtime
    x = _integer_patterns(22, 37 * 129)
    y = _integer_patterns(23, 37 * 129)[::-1].copy()
    y[::5] = x[::5]                                        # equal operands for the comparisons
    want = numpy_ops.integer_binary(name, x, y)
    x_d, y_d, z_d = rt.array(x.view(f32)), rt.array(y.view(f32)), rt.empty(x.shape)
    sb = FusedSpecBuilder(x.shape)
    tx, ty, tz = sb.tensor(x_d.ptr, [1]), sb.tensor(y_d.ptr, [1]), sb.tensor(z_d.ptr, [1])
    sb.store(tz, sb.binary(name, sb.load(tx), sb.load(ty)))
    rt.launch_fused(sb.build())
    got = z_d.get()
    for d in (x_d, y_d, z_d):
        d.free()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("name", ["sum", "prod", "max", "min", "argmax", "argmin"])
@pytest.mark.parametrize("shape,layout", [((64, 10), "row"), ((64, 10), "col"), ((5000, 3), "row"),
                                          ((300, 700), "col"), ((1, 9), "row"), ((40000, 2), "col"),
                                          # many columns: the whole workgroup lies along them
                                          ((300, 4096), "col"), ((37, 4100), "col"), ((2000, 1027), "col"),
                                          # thousands of rows of a few hundred chunks: a wavefront per row
                                          ((1024, 4200), "row"), ((300, 5000), "row"), ((401, 4100), "row"),
                                          ((2048, 4096), "row"),
                                          # rows that are not whole float4s: 4 elements per lane all the same,
                                          # a short last chunk per row (several rows per workgroup, a wavefront
                                          # per row, a workgroup per row, several workgroups per row)
                                          ((77, 300), "row"), ((1001, 4200), "row"), ((4099, 40), "row"),
                                          ((20003, 5), "row")])
def test_every_reduction(hip_runtime, name, shape, layout):
    """Reduce axis 0 of an [R, A] view; 'row' = R contiguous in memory, 'col' = A contiguous."""
    rt = hip_runtime
    R, A = shape
    rs = np.random.RandomState(13)
    scale = 0.05 if name == "prod" else 1.0
    if name == "prod":
        logical = (1.0 + rs.normal(0, scale, (R, A))).astype(f32)
    elif name == "sum":
        # same-sign data: a relative bound on the result is meaningful (a signed sum
        # cancels and is checked against float64 in test_signed_sum_against_float64)
        logical = rs.uniform(0.5, 1.5, (R, A)).astype(f32)
    else:
        logical = rs.normal(0, 1, (R, A)).astype(f32)
    if name in ("argmax", "argmin", "max", "min") and R > 3:
        logical[R // 2] = logical[R // 3]           # ties: lowest index must win
    want = numpy_ops.reduce(name, logical, 0)
    if layout == "row":
        store, strides = np.ascontiguousarray(logical.T), [1, R]
    else:
        store, strides = logical, [A, 1]
    x_d = rt.array(store)
    is_arg = name.startswith("arg")
    out_d = rt.empty((A,), NGH_I32 if is_arg else NGH_F32)
    sb = FusedSpecBuilder([R, A])
    tx = sb.tensor(x_d.ptr, strides)
    to = sb.tensor(out_d.ptr, [0, 1], NGH_I32 if is_arg else NGH_F32)
    sb.reduce(name, sb.load(tx), to)
    spec = sb.build()
    rt.launch_fused(spec)
    got = out_d.get()
    if layout == "row" and R % 4 and R >= 8 and name == "sum" and default_kernel_choice():
        assert rt.describe_fused(spec, 0).endswith("/ragged")
    if is_arg:
        np.testing.assert_array_equal(got, want)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5 if name != "prod" else 1e-4, atol=1e-5)
    x_d.free()
    out_d.free()


@pytest.mark.parametrize("layout", ["row", "col"])
@pytest.mark.parametrize("name", ["sum", "prod", "max", "min", "argmax", "argmin"])
def test_reductions_over_nan_and_infinities(hip_runtime, name, layout):
    """Columns holding a NaN, infinities of one sign, of both signs, or only finite values:
    np.sum / prod / max / min give NaN for a column with a NaN (and sum for +inf with -inf),
    np.argmax / argmin the position of the first NaN (cputransform.py:521-527, 670-676)."""
    rt = hip_runtime
    R, A = 700, 12
    rs = np.random.RandomState(21)
    logical = rs.uniform(0.5, 1.5, (R, A)).astype(f32)
    logical[300, 1] = np.nan
    logical[5, 2] = np.nan
    logical[650, 2] = np.nan
    logical[100, 3] = np.inf
    logical[101, 4] = -np.inf
    logical[10, 5] = np.inf
    logical[600, 5] = -np.inf
    logical[0, 6] = np.nan
    logical[R - 1, 7] = np.nan
    logical[200, 8] = np.inf
    logical[400, 8] = np.nan
    logical[50, 9] = np.inf
    logical[60, 9] = np.inf
    want = numpy_ops.reduce(name, logical, 0)
    store, strides = (np.ascontiguousarray(logical.T), [1, R]) if layout == "row" else (logical, [A, 1])
    x_d = rt.array(store)
    is_arg = name.startswith("arg")
    out_d = rt.empty((A,), NGH_I32 if is_arg else NGH_F32)
    sb = FusedSpecBuilder([R, A])
    tx = sb.tensor(x_d.ptr, strides)
    to = sb.tensor(out_d.ptr, [0, 1], NGH_I32 if is_arg else NGH_F32)
    sb.reduce(name, sb.load(tx), to)
    rt.launch_fused(sb.build())
    got = out_d.get()
    x_d.free()
    out_d.free()
    if is_arg:
        np.testing.assert_array_equal(got, want)
    else:
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
        np.testing.assert_allclose(got[~np.isnan(want)], want[~np.isnan(want)], rtol=1e-4)


@pytest.mark.parametrize("name", ["sum", "max", "min", "argmax", "argmin"])
@pytest.mark.parametrize("shape,layout", [((1 << 20, 3), "row"), ((1 << 20, 4), "col"), ((1 << 21, 1), "row")])
def test_reductions_into_a_handful_of_outputs_with_hundreds_of_segments(hip_runtime, name, shape, layout):
    """A few outputs, each split into 256 segments or more: the merge takes a workgroup per
    output.  Ties across segments (the lowest index wins) and a NaN in one segment included."""
    from ngraph_hip.runtime.hiplib import plan_fused
    rt = hip_runtime
    R, A = shape
    rs = np.random.RandomState(15)
    logical = (rs.uniform(0.5, 1.5, (R, A)) if name == "sum" else rs.normal(0, 1, (R, A))).astype(f32)
    if name != "sum":
        extreme = f32(9.0 if name in ("max", "argmax") else -9.0)
        logical[R // 3, :] = extreme                   # the same extreme value in two far-apart segments
        logical[R // 3 * 2, :] = extreme
        if name in ("max", "min"):
            logical[R // 2, A - 1] = np.nan            # ... and a NaN in the last output's rows
    want = numpy_ops.reduce(name, logical, 0)
    if layout == "row":
        store, strides = np.ascontiguousarray(logical.T), [1, R]
    else:
        store, strides = logical, [A, 1]
    x_d = rt.array(store)
    is_arg = name.startswith("arg")
    out_d = rt.empty((A,), NGH_I32 if is_arg else NGH_F32)
    sb = FusedSpecBuilder([R, A])
    sb.reduce(name, sb.load(sb.tensor(x_d.ptr, strides)), sb.tensor(out_d.ptr, [0, 1], NGH_I32 if is_arg else NGH_F32))
    spec = sb.build()
    if default_kernel_choice():
        assert plan_fused(spec)["segments"] >= 256
    rt.launch_fused(spec)
    got = out_d.get()
    if is_arg:
        np.testing.assert_array_equal(got, want)
    else:
        np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        if name == "sum":
            # a million same-sign terms: the oracle's ufunc adds the rows of a C-ordered operand one
            # after the other in float32 and drifts by up to 2e-5 of the result; float64 decides,
            # and the device's segments and tree are the closer side
            truth = logical.astype(np.float64).sum(axis=0)
            np.testing.assert_allclose(got, truth, rtol=2e-6)
            np.testing.assert_allclose(want, truth, rtol=1e-4)
        else:
            np.testing.assert_allclose(got[ok], want[ok], rtol=1e-5)
    x_d.free()
    out_d.free()


@pytest.mark.parametrize("name", ["argmax", "argmin"])
def test_arg_reduction_index_beyond_2_to_24_is_exact(hip_runtime, name):
    """An index above 2^24 reaches int32 storage as the integer it is (no trip through an fp32
    register, which would round it to an even number); the same reduction into fp32 is refused."""
    from ngraph_hip.runtime.hiplib import HipLibraryError
    rt = hip_runtime
    R = (1 << 24) + 1025
    x = np.zeros((R, 1), f32)
    where = [(1 << 24) + 1001]                    # odd, above 2^24: not an fp32 number
    x[where[0], 0] = 5.0 if name == "argmax" else -5.0
    x_d = rt.array(x)
    out_d, out_f = rt.empty((1,), NGH_I32), rt.empty((1,))
    for layout in ([1, 1], [1, R]):               # as a column and as a row
        rt.memset32(out_d.ptr, 0, 1)
        sb = FusedSpecBuilder([R, 1])
        sb.reduce(name, sb.load(sb.tensor(x_d.ptr, layout)), sb.tensor(out_d.ptr, [0, 1], NGH_I32))
        rt.launch_fused(sb.build())
        assert out_d.get().tolist() == where
    sb = FusedSpecBuilder([R, 1])
    sb.reduce(name, sb.load(sb.tensor(x_d.ptr, [1, 1])), sb.tensor(out_f.ptr, [0, 1]))
    with pytest.raises(HipLibraryError) as e:
        rt.launch_fused(sb.build())
    assert e.value.code == -4
    for d in (x_d, out_d, out_f):
        d.free()


@pytest.mark.parametrize("shape,layout", [((40000, 2), "col"), ((200704, 4), "row"), ((3000, 300), "col"),
                                          ((3000, 2048), "col")])
def test_signed_sum_against_float64(hip_runtime, shape, layout):
    """A cancelling sum: error must stay within 1e-6 of sum(|x|), checked against float64."""
    rt = hip_runtime
    R, A = shape
    rs = np.random.RandomState(14)
    logical = rs.normal(0.5, 2, (R, A)).astype(f32)
    truth = logical.astype(np.float64).sum(axis=0)
    bound = 1e-6 * np.abs(logical).astype(np.float64).sum(axis=0)
    if layout == "row":
        store, strides = np.ascontiguousarray(logical.T), [1, R]
    else:
        store, strides = logical, [A, 1]
    x_d, out_d = rt.array(store), rt.empty((A,))
    sb = FusedSpecBuilder([R, A])
    tx, to = sb.tensor(x_d.ptr, strides), sb.tensor(out_d.ptr, [0, 1])
    sb.reduce("sum", sb.load(tx), to)
    rt.launch_fused(sb.build())
    assert np.all(np.abs(out_d.get().astype(np.float64) - truth) <= bound)
    x_d.free()
    out_d.free()


@pytest.mark.parametrize("R,A", [(512, 2048), (100, 4100), (64, 1024), (1500, 1027)])
def test_column_reductions_with_elementwise_stores_over_many_columns(hip_runtime, R, A):
    """z = tanh(x*y + 0.5) stored, max and argmax of z and sum of x*x down the columns, in one
    stage over [R, A] with A contiguous: every lane of the workgroup owns its columns, rows are
    split into segments, and the plan reports it (family 2)."""
    from ngraph_hip.runtime.hiplib import plan_fused
    rt = hip_runtime
    rs = np.random.RandomState(R + A)
    x, y = rs.normal(0, 1, (R, A)).astype(f32), rs.normal(0, 1, (R, A)).astype(f32)
    x[R // 2] = x[R // 3]
    y[R // 2] = y[R // 3]                                  # ties: the lowest index wins
    x_d, y_d, z_d = rt.array(x), rt.array(y), rt.empty((R, A))
    mx_d, am_d, ss_d = rt.empty((A,)), rt.empty((A,), NGH_I32), rt.empty((A,))
    sb = FusedSpecBuilder([R, A])
    tx, ty, tz = (sb.tensor(d.ptr, [A, 1]) for d in (x_d, y_d, z_d))
    tmx, tss = sb.tensor(mx_d.ptr, [0, 1]), sb.tensor(ss_d.ptr, [0, 1])
    tam = sb.tensor(am_d.ptr, [0, 1], NGH_I32)
    rx, ry = sb.load(tx), sb.load(ty)
    z = sb.unary("tanh", sb.binary("add", sb.binary("mul", rx, ry), sb.constant(0.5)))
    sb.store(tz, z)
    sq = sb.unary("sqr", rx)
    sb.reduce("max", z, tmx)
    sb.reduce("argmax", z, tam)
    sb.reduce("sum", sq, tss)
    spec = sb.build()
    assert plan_fused(spec)["family"] == 2
    rt.launch_fused(spec)
    z_w = numpy_ops.unary("tanh", numpy_ops.binary("add", numpy_ops.binary("mul", x, y), f32(0.5)))
    z_g = z_d.get()
    np.testing.assert_allclose(z_g, z_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_array_equal(mx_d.get(), z_g.max(axis=0))
    np.testing.assert_array_equal(am_d.get(), z_g.argmax(axis=0))
    np.testing.assert_allclose(ss_d.get(), (x.astype(np.float64) ** 2).sum(axis=0), rtol=RTOL, atol=ATOL)
    for d in (x_d, y_d, z_d, mx_d, am_d, ss_d):
        d.free()


# ------------------------------------------------------------------ one-pass moments
@pytest.mark.parametrize("rows,R,pad", [(1, 1, 3), (3, 2, 2), (5, 7, 1), (4, 1024, 0), (256, 3136, 0),
                                        (2, 1000003, 1), (700, 260, 0), (1, 4, 0),
                                        # many short rows: a wavefront per row
                                        (4096, 1024, 0), (5000, 1027, 1), (70000, 3, 1), (4100, 4096, 0),
                                        (4100, 4100, 0)])
def test_moments_rows(hip_runtime, rows, R, pad):
    """ngh_moments_f32 against float64 row statistics; rows of every length class (shorter than
    a vector, ragged tails, many segments, thousands of short rows), with a row stride wider than the row.  Launched
    twice: the second launch checks that the arrival counters were left at zero."""
    rt = hip_runtime
    rs = np.random.RandomState(rows * 7 + R)
    stride = ((R + 3) // 4) * 4 + 4 * pad
    host = rs.normal(3.0, 2.0, (rows, stride)).astype(f32)
    x_d = rt.array(host)
    out_d = rt.empty((3, rows))
    eps = 1e-5
    x64 = host[:, :R].astype(np.float64)
    for _ in range(2):
        rt.memset32(out_d.ptr, 0, 3 * rows)
        rt.moments_f32(x_d.ptr, rows, R, stride, out_d.ptr, out_d.ptr + 4 * rows, out_d.ptr + 8 * rows, eps)
        mean, var, rstd = out_d.get()
        np.testing.assert_allclose(mean, x64.mean(axis=1), rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(var, x64.var(axis=1), rtol=1e-4, atol=1e-5)
        # rstd is the fp32 statement sequence add, sqrt, reciprocal on the kernel's own variance
        want = (f32(1) / np.sqrt(var + f32(eps))).astype(f32)
        np.testing.assert_array_equal(rstd, want)
    # without rstd the third row stays untouched
    rt.memset32(out_d.ptr, 0, 3 * rows)
    rt.moments_f32(x_d.ptr, rows, R, stride, out_d.ptr, out_d.ptr + 4 * rows)
    assert not out_d.get()[2].any()
    for d in (x_d, out_d):
        d.free()


@pytest.mark.parametrize("rows,R,stride,first", [(256, 3137, 3139, 1), (5000, 1001, 1001, 3), (37, 100003, 100005, 2),
                                                 (4100, 4095, 4097, 1), (70000, 5, 7, 1)])
def test_moments_of_rows_off_16_byte_boundaries(hip_runtime, rows, R, stride, first):
    """Rows that start at any float: odd row pitch, a view that begins a few elements into its
    buffer.  Both kernels (segments of long rows, a group of lanes per short row) read them with
    unaligned 16-byte loads; results against float64."""
    rt = hip_runtime
    rs = np.random.RandomState(rows + R)
    host = rs.normal(-1.0, 3.0, first + rows * stride).astype(f32)
    x_d = rt.array(host)
    out_d = rt.empty((3, rows))
    rt.memset32(out_d.ptr, 0x7fc00000, 3 * rows)
    rt.moments_f32(x_d.ptr + 4 * first, rows, R, stride, out_d.ptr, out_d.ptr + 4 * rows, out_d.ptr + 8 * rows, 1e-5)
    mean, var, rstd = out_d.get()
    view = np.lib.stride_tricks.as_strided(host[first:], (rows, R), (4 * stride, 4)).astype(np.float64)
    np.testing.assert_allclose(mean, view.mean(axis=1), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var, view.var(axis=1), rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(rstd, (f32(1) / np.sqrt(var + f32(1e-5))).astype(f32))
    for d in (x_d, out_d):
        d.free()


def test_moments_hand_off_with_and_without_release_acquire_tickets(monkeypatch):
    """A row's segments are merged in segment order.  By default the moments kernel ends after
    writing its partial sums and a second small launch merges them (the kernel boundary is the
    hand-off).  NGH_ORDERED_ARRIVAL=0 / 1 merge inside the one launch, in the last workgroup of
    the row to finish: 0 hands over with a relaxed ticket ordered behind the partial sums by a
    data dependency (what gfx950 honours), 1 with release tickets and an acquire fence in the
    merger (what the memory model asks of one launch, at 2.6 times the kernel's duration).  Same
    sums in the same order: identical results."""
    from ngraph_hip.runtime.hiplib import HipRuntime
    rs = np.random.RandomState(21)
    x = rs.normal(3.0, 2.0, (300, 50000)).astype(f32)
    seen = []
    for ordered in (None, "2", "0", "1"):
        monkeypatch.delenv("NGH_ORDERED_ARRIVAL", raising=False)
        if ordered is not None:
            monkeypatch.setenv("NGH_ORDERED_ARRIVAL", ordered)
        rt = HipRuntime(0)
        try:
            x_d, out_d = rt.array(x), rt.empty((3, 300))
            for _ in range(3):                       # the arrival counters must be left at zero each time
                rt.memset32(out_d.ptr, 0, 900)
                rt.moments_f32(x_d.ptr, 300, 50000, 50000, out_d.ptr, out_d.ptr + 1200, out_d.ptr + 2400, 1e-5)
                seen.append(out_d.get())
        finally:
            rt.close()
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(seen[0][0], x64.mean(axis=1), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(seen[0][1], x64.var(axis=1), rtol=RTOL, atol=ATOL)
    for other in seen[1:]:
        np.testing.assert_array_equal(other, seen[0])


# ------------------------------------------------------------------ tiled skeleton (transposed views)
def _transpose_program(rt, shape3, x_d, y_d, z_d, w_d, in_place):
    """Over logical [O, A, B]:  y[o,a,b] (B-contiguous) = 2*x[o,b,a]^T + z[o,a,b];
    w[o,b,a] (A-contiguous, i.e. a transposed output) = y - 1; with in_place, x is overwritten
    by w instead."""
    O, A, B = shape3
    sb = FusedSpecBuilder([O, A, B])
    tx = sb.tensor(x_d.ptr, [A * B, 1, A])        # x stored [O, B, A]: contiguous along A
    tz = sb.tensor(z_d.ptr, [A * B, B, 1])        # z stored [O, A, B]
    ty = sb.tensor(y_d.ptr, [A * B, B, 1])
    tw = tx if in_place else sb.tensor(w_d.ptr, [A * B, 1, A])
    x = sb.load(tx)
    z = sb.load(tz)
    y = sb.binary("add", sb.binary("mul", x, sb.constant(2.0)), z)
    sb.store(ty, y)
    sb.store(tw, sb.binary("sub", y, sb.constant(1.0)))
    return sb.build()


@pytest.mark.parametrize("shape3", [(1, 64, 64), (1, 1024, 64), (3, 50, 37), (2, 33, 200), (1, 9, 8), (1, 2048, 2048)])
@pytest.mark.parametrize("in_place", [False, True])
def test_tiled_transposed_operands(hip_runtime, shape3, in_place):
    """Inputs and outputs of both orientations in one stage: the planner picks the LDS-tiled
    skeleton (family 3) and every element lands where the strided views say."""
    from ngraph_hip.runtime import hiplib
    rt = hip_runtime
    O, A, B = shape3
    rs = np.random.RandomState(A * 31 + B)
    x = rs.normal(0, 1, (O, B, A)).astype(f32)
    z = rs.normal(0, 1, (O, A, B)).astype(f32)
    x_d, z_d = rt.array(x), rt.array(z)
    y_d, w_d = rt.empty((O, A, B)), rt.empty((O, B, A))
    spec = _transpose_program(rt, shape3, x_d, y_d, z_d, w_d, in_place)
    assert hiplib.plan_fused(spec, 0)["family"] == 3
    if default_kernel_choice():
        assert rt.describe_fused(spec, 0).startswith("ew_tiled_interp")
    rt.launch_fused(spec)
    y_w = (x.transpose(0, 2, 1) * f32(2.0) + z).astype(f32)
    w_w = (y_w - f32(1.0)).transpose(0, 2, 1)
    np.testing.assert_array_equal(y_d.get(), y_w)
    np.testing.assert_array_equal((x_d if in_place else w_d).get(), w_w)
    for d in (x_d, z_d, y_d, w_d):
        d.free()


def test_tiled_flex_transposed_output_with_statistics(hip_runtime):
    """A flex16 result written through a transposed view: quantisation and max|mantissa| happen
    at the staged store."""
    from ngraph_hip.runtime import NGH_FLEX16
    from oracle import flex_model as fm
    rt = hip_runtime
    A, B = 70, 45
    rs = np.random.RandomState(5)
    x = rs.normal(0, 1, (A, B)).astype(f32)
    x_d = rt.array(x)
    y_d = rt.empty((B, A), NGH_FLEX16)
    stats = rt.stats_alloc(1)
    dec = 12
    sb = FusedSpecBuilder([A, B])
    tx = sb.tensor(x_d.ptr, [B, 1])
    ty = sb.tensor(y_d.ptr, [1, A], NGH_FLEX16, scale=2.0 ** -dec, dev_stats=stats)
    sb.store(ty, sb.binary("mul", sb.load(tx), sb.constant(3.0)))
    spec = sb.build()
    if default_kernel_choice():
        assert rt.describe_fused(spec, 0).startswith("ew_tiled_interp")
    rt.launch_fused(spec)
    want = fm.quantize_rni((x * f32(3.0)).T, dec)
    np.testing.assert_array_equal(y_d.get(), want)
    assert int(rt.stats_read(stats, 1)[0]) == fm.maxabs(want)
    for d in (x_d, y_d):
        d.free()
    rt.free(stats)


# ------------------------------------------------------------------ take (table lookup)
@pytest.mark.parametrize("lut_axis", [0, 1])
@pytest.mark.parametrize("I,F,V", [(37, 24, 50), (1000, 256, 300), (5, 3, 2)])
def test_take_lookup(hip_runtime, lut_axis, I, F, V):
    """NGH_OP_TAKE against ndarray.take; indices outside the table are clamped to it."""
    rt = hip_runtime
    rs = np.random.RandomState(I + F)
    lut = rs.normal(0, 1, (V, F) if lut_axis == 0 else (F, V)).astype(f32)
    idx = rs.randint(0, V, I).astype(f32)
    idx[0], idx[-1] = -3.0, V + 7.0                       # out of range on both sides
    lut_d, idx_d = rt.array(lut), rt.array(idx)
    if lut_axis == 0:          # out[i, f] = lut[idx[i], f]
        shape, idx_st, lut_st, out_st, axis = [I, F], [1, 0], [F, 1], [F, 1], 0
    else:                      # out[f, i] = lut[f, idx[i]]
        shape, idx_st, lut_st, out_st, axis = [F, I], [0, 1], [V, 1], [I, 1], 1
    out_d = rt.empty(shape)
    sb = FusedSpecBuilder(shape)
    ti = sb.tensor(idx_d.ptr, idx_st)
    tl = sb.tensor(lut_d.ptr, lut_st, take_extent=V)
    to = sb.tensor(out_d.ptr, out_st)
    sb.store(to, sb.take(tl, sb.load(ti), axis))
    rt.launch_fused(sb.build())
    want = lut.take(np.clip(idx, 0, V - 1).astype(int), lut_axis)
    np.testing.assert_array_equal(out_d.get(), want)
    for d in (lut_d, idx_d, out_d):
        d.free()


@pytest.mark.parametrize("N,V", [(37, 50), (1000003, 50), (19, 3)])
def test_take_lookup_along_a_single_axis_with_a_scalar_tail(hip_runtime, N, V):
    """out[i] = lut[idx[i]] as a 1-D stage whose length is not a multiple of the vector width:
    the vector body and the scalar tail both index the table from its first element."""
    rt = hip_runtime
    rs = np.random.RandomState(N)
    lut = rs.normal(0, 1, V).astype(f32)
    idx = rs.randint(0, V, N).astype(f32)
    idx[-3:] = [V - 1, V - 2, V + 5]                      # the tail reads the table's end
    idx[0] = -2.0
    lut_d, idx_d, out_d = rt.array(lut), rt.array(idx), rt.empty((N,))
    sb = FusedSpecBuilder([N])
    ti = sb.tensor(idx_d.ptr, [1])
    tl = sb.tensor(lut_d.ptr, [1], take_extent=V)
    to = sb.tensor(out_d.ptr, [1])
    sb.store(to, sb.take(tl, sb.load(ti), 0))
    spec = sb.build()
    from ngraph_hip.runtime.hiplib import plan_fused
    assert plan_fused(spec)["tail"] == N % 4
    rt.launch_fused(spec)
    np.testing.assert_array_equal(out_d.get(), lut.take(np.clip(idx, 0, V - 1).astype(int)))
    for d in (lut_d, idx_d, out_d):
        d.free()


def test_iota_along_a_single_axis_with_a_scalar_tail(hip_runtime):
    """The index value of an element in the tail is its index in the whole view."""
    rt = hip_runtime
    n = 4099
    y_d = rt.empty((n,))
    sb = FusedSpecBuilder([n])
    ty = sb.tensor(y_d.ptr, [1])
    sb.store(ty, sb.iota(0))
    rt.launch_fused(sb.build())
    np.testing.assert_array_equal(y_d.get(), np.arange(n, dtype=f32))
    y_d.free()


def test_take_needs_an_extent(hip_runtime):
    from ngraph_hip.runtime.hiplib import HipLibraryError
    rt = hip_runtime
    lut_d, idx_d, out_d = rt.empty((4, 4)), rt.empty((3,)), rt.empty((3, 4))
    sb = FusedSpecBuilder([3, 4])
    ti, tl, to = sb.tensor(idx_d.ptr, [1, 0]), sb.tensor(lut_d.ptr, [4, 1]), sb.tensor(out_d.ptr, [4, 1])
    sb.store(to, sb.take(tl, sb.load(ti), 0))
    with pytest.raises(HipLibraryError):
        rt.launch_fused(sb.build())
    for d in (lut_d, idx_d, out_d):
        d.free()


def test_truncating_store_is_the_flex_fill_rule(hip_runtime):
    """STORE_TRUNC: mantissa = int(value / scale) cut toward zero and clipped
    (tensor_ops.py:690-707), where the ordinary store rounds to nearest."""
    from ngraph_hip.runtime import NGH_FLEX16
    rt = hip_runtime
    n, dec = 1000, 14
    values = [1.2, -1.2, 0.99999, 5.0, -5.0]               # the last two saturate at dec 14
    for value in values:
        for truncate in (True, False):
            y_d = rt.empty((n,), NGH_FLEX16)
            stats = rt.stats_alloc(1)
            sb = FusedSpecBuilder([n])
            ty = sb.tensor(y_d.ptr, [1], NGH_FLEX16, scale=2.0 ** -dec, dev_stats=stats)
            sb.store(ty, sb.constant(value), truncate=truncate)
            rt.launch_fused(sb.build())
            scaled = np.float32(value) * np.float32(2.0 ** dec)
            want = int(np.clip(np.trunc(scaled) if truncate else np.rint(scaled), -32768, 32767))
            got = y_d.get()
            assert (got == want).all(), (value, truncate, got[:4], want)
            assert int(rt.stats_read(stats, 1)[0]) == abs(want)
            y_d.free()
            rt.free(stats)


def test_rng_is_a_function_of_seed_counter_and_element(hip_runtime):
    """The random fill draws per element from (seed, counter, linear index, stream): the same
    numbers come out whatever the launch shape, and a new counter or seed gives new ones."""
    rt = hip_runtime
    A, B = 96, 1000

    def draw(shape, strides, seed, counter, dist="uniform"):
        y_d = rt.empty((A * B,))
        sb = FusedSpecBuilder(shape)
        ty = sb.tensor(y_d.ptr, strides)
        sb.store(ty, sb.rng(dist, 0))
        spec = sb.build()
        spec.rng_seed, spec.rng_counter = seed, counter
        rt.launch_fused(spec)
        out = y_d.get()
        y_d.free()
        return out

    flat = draw([A * B], [1], 7, 0)                         # one contiguous axis: vector stores
    two_d = draw([A, B], [B, 1], 7, 0)                      # same elements as a matrix
    transposed = draw([B, A], [1, B], 7, 0)                 # walked column by column
    np.testing.assert_array_equal(flat, two_d)
    # the transposed walk numbers element (b, a) as b * A + a: the same set, permuted
    np.testing.assert_array_equal(np.sort(transposed), np.sort(flat))
    np.testing.assert_array_equal(transposed.reshape(A, B).T.ravel(), flat)
    assert flat.min() >= 0.0 and flat.max() < 1.0 and abs(flat.mean() - 0.5) < 0.01
    assert not np.array_equal(flat, draw([A * B], [1], 7, 1))
    assert not np.array_equal(flat, draw([A * B], [1], 8, 0))
    np.testing.assert_array_equal(flat, draw([A * B], [1], 7, 0))
    z = draw([A * B], [1], 7, 0, "normal")
    assert abs(z.mean()) < 0.02 and abs(z.std() - 1.0) < 0.02
    # a length that leaves a scalar tail: element i draws what element i of any longer or
    # shorter fill draws, so the tail continues the body's sequence instead of restarting it
    n = A * B - 5
    y_d = rt.empty((n,))
    sb = FusedSpecBuilder([n])
    sb.store(sb.tensor(y_d.ptr, [1]), sb.rng("uniform", 0))
    spec = sb.build()
    spec.rng_seed, spec.rng_counter = 7, 0
    rt.launch_fused(spec)
    odd = y_d.get()
    y_d.free()
    assert n % 4 == 3
    np.testing.assert_array_equal(odd, flat[:n])
    assert not np.array_equal(odd[-3:], odd[:3])


@pytest.mark.parametrize("n", [4096, 100003])
def test_convert_between_fp32_and_flex16(hip_runtime, n):
    """Storage types may differ inside one kernel: fp32 -> flex16 is the quantising conversion
    (round to nearest even, saturate, max|mantissa|), flex16 -> fp32 the dequantisation."""
    from ngraph_hip.runtime import NGH_FLEX16
    from oracle import flex_model as fm
    rt = hip_runtime
    rs = np.random.RandomState(n)
    x = rs.normal(0, 3.0, n).astype(f32)
    dec = 12                                               # +-8 range: some elements saturate
    x_d, q_d, back_d = rt.array(x), rt.empty((n,), NGH_FLEX16), rt.empty((n,))
    stats = rt.stats_alloc(1)
    sb = FusedSpecBuilder([n])
    sb.store(sb.tensor(q_d.ptr, [1], NGH_FLEX16, scale=2.0 ** -dec, dev_stats=stats), sb.load(sb.tensor(x_d.ptr, [1])))
    rt.launch_fused(sb.build())
    want = fm.quantize_rni(x, dec)
    np.testing.assert_array_equal(q_d.get(), want)
    assert int(rt.stats_read(stats, 1)[0]) == fm.maxabs(want)
    sb = FusedSpecBuilder([n])
    sb.store(sb.tensor(back_d.ptr, [1]), sb.load(sb.tensor(q_d.ptr, [1], NGH_FLEX16, scale=2.0 ** -dec)))
    rt.launch_fused(sb.build())
    np.testing.assert_array_equal(back_d.get(), fm.dequantize(want, dec))
    for d in (x_d, q_d, back_d):
        d.free()
    rt.free(stats)


INT_TYPES = [("NGH_I32", np.int32), ("NGH_U32", np.uint32), ("NGH_I16", np.int16), ("NGH_I8", np.int8),
             ("NGH_U8", np.uint8)]


@pytest.mark.parametrize("type_name,np_type", INT_TYPES)
@pytest.mark.parametrize("shape", [(4096,), (7, 33), (3, 64, 48)])
def test_integer_storage_types(hip_runtime, type_name, np_type, shape):
    """Integer tensors are converted to float on load and back on store (float_ew2.py:615-641
    declares the same storage types).  A store truncates toward zero and saturates at the
    type's range; inside the range that is NumPy's astype, which is what the CPU transformer
    does."""
    import ngraph_hip.runtime as runtime
    code = getattr(runtime, type_name)
    rt = hip_runtime
    info = np.iinfo(np_type)
    lo, hi = max(info.min, -(1 << 20)), min(info.max, 1 << 20)      # exact in fp32
    rs = np.random.RandomState(len(shape) + info.bits)
    src = rs.randint(lo, hi + 1, size=shape).astype(np_type)
    x = rs.uniform(-1.5, 1.5, size=shape).astype(f32) * f32(min(hi, 1 << 15))
    st = contiguous_strides(shape)
    src_d, x_d = rt.array(src, code), rt.array(x)
    as_float_d, as_int_d = rt.empty(shape), rt.empty(shape, code)
    sb = FusedSpecBuilder(shape)
    v = sb.load(sb.tensor(src_d.ptr, st, code))
    sb.store(sb.tensor(as_float_d.ptr, st), sb.binary("mul", v, sb.constant(0.5)))
    sb.store(sb.tensor(as_int_d.ptr, st, code), sb.load(sb.tensor(x_d.ptr, st)))
    rt.launch_fused(sb.build())
    np.testing.assert_array_equal(as_float_d.get(), src.astype(f32) * f32(0.5))
    want = np.clip(np.trunc(x.astype(np.float64)), info.min, info.max).astype(np_type)
    np.testing.assert_array_equal(as_int_d.get(), want)
    inside = (x > info.min) & (x < info.max)
    np.testing.assert_array_equal(as_int_d.get()[inside], x[inside].astype(np_type))
    for d in (src_d, x_d, as_float_d, as_int_d):
        d.free()


@pytest.mark.parametrize("np_type", [np.int8, np.uint8])
def test_byte_views_copy(hip_runtime, np_type):
    """The strided copy moves 1-byte elements too (transposed and sliced views)."""
    rt = hip_runtime
    rs = np.random.RandomState(5)
    src = rs.randint(0, 100, size=(70, 130)).astype(np_type)
    import ngraph_hip.runtime as runtime
    code = runtime.NGH_I8 if np_type is np.int8 else runtime.NGH_U8
    src_d, dst_d = rt.array(src), rt.empty((130, 70), code)
    rt.copy_strided(dst_d.ptr, src_d.ptr, (130, 70), (70, 1), (1, 130), 1)
    np.testing.assert_array_equal(dst_d.get(), src.T)
    src_d.free()
    dst_d.free()


def test_flex_ids_past_the_end_of_the_table_are_rejected(hip_runtime):
    """Record numbers are checked against the table they index before any kernel runs."""
    from ngraph_hip.runtime.hiplib import HipLibraryError
    rt = hip_runtime
    table = rt.flex_states_alloc(3)
    try:
        rt.flex_prepare(table, [0, 2], [0, 0])
        rt.flex_update(table, [2], 1)
        for bad in ([3], [0, 7], [1 << 20]):
            with pytest.raises(HipLibraryError) as e:
                rt.flex_prepare(table, bad, [0] * len(bad))
            assert e.value.code == -1
            with pytest.raises(HipLibraryError):
                rt.flex_update(table, bad, 1)
        # counted from a record inside the table: two records are left after the first
        with pytest.raises(HipLibraryError):
            rt.flex_update(table + 168, [2], 1)
        rt.flex_update(table + 168, [1], 1)
        rt.sync()
    finally:
        rt.free(table)


@pytest.mark.parametrize("src", ["f32", "f16"])
@pytest.mark.parametrize("n,offset", [(1 << 20, 0), (100003, 0), (4099, 1), (5, 0), (1 << 22, 0)])
def test_truncating_converter_to_flex16(hip_runtime, src, n, offset):
    """ngh_convert_to_flex16 against the statement of the reference's `convert` kernel
    (gpu/flex_conv.py:745-791): mantissa = (short)(value * scale), i.e. truncation toward zero,
    max |mantissa| merged into the statistics word.  Outside the int16 range, where that cast
    is undefined, the library saturates; NaN gives 0.  `offset` starts the views off the
    16-byte boundary (the scalar path)."""
    from ngraph_hip.runtime.hiplib import NGH_FLEX16, NGH_F16
    rt = hip_runtime
    rs = np.random.RandomState(n + offset)
    np_src = np.float32 if src == "f32" else np.float16
    dec = 9
    values = rs.normal(0, 8, n + offset).astype(np_src)
    values[offset:offset + 5] = np.array([1.999, -1.999, 63.99, -64.0, 0.0009765625], np_src)[:min(5, n)]
    if n > 100:
        values[offset + 50:offset + 54] = [70.0, -70.0, np.inf, -np.inf]      # beyond int16 at dec 9: saturate
        values[offset + 60] = np.nan
    src_d = rt.array(values, NGH_F32 if src == "f32" else NGH_F16)
    out_d = rt.empty((n + offset,), NGH_FLEX16)
    rt.memset16(out_d.ptr, 0x7777, n + offset)
    stats = rt.stats_alloc(1)
    itemsize = values.dtype.itemsize
    rt.convert_to_flex16(out_d.ptr + 2 * offset, src_d.ptr + itemsize * offset, NGH_F32 if src == "f32" else NGH_F16,
                         n, scale=float(2 ** dec), dev_stats=stats)
    got = out_d.get()
    with np.errstate(all="ignore"):
        scaled = values[offset:].astype(np.float32) * np.float32(2 ** dec)           # cvt(value) * scale in fp32
        want = np.clip(np.trunc(np.where(np.isnan(scaled), 0, scaled)), -32768, 32767).astype(np.int16)
    np.testing.assert_array_equal(got[offset:], want)
    assert (got[:offset] == 0x7777).all()                                           # nothing before the view
    assert rt.stats_read(stats, 1)[0] == int(np.abs(want.astype(np.int32)).max())
    # truncation, not rounding: 1.999 * 512 = 1023.49 -> 1023 and -1.999 -> -1023, 63.99 * 512 = 32762.9 -> 32762
    if n >= 5:
        first = (np.array([1.999, -1.999, 63.99], np_src).astype(np.float32) * 512).astype(np.float64)
        assert got[offset:offset + 3].tolist() == np.clip(np.trunc(first), -32768, 32767).astype(int).tolist()
    # the multiplier read from a device word (the tensor's scale 2**-dec) gives the same mantissas
    scale_d = rt.array(np.array([2.0 ** -dec], np.float32))
    rt.memset16(out_d.ptr, 0, n + offset)
    rt.convert_to_flex16(out_d.ptr + 2 * offset, src_d.ptr + itemsize * offset, NGH_F32 if src == "f32" else NGH_F16,
                         n, scale=123.0, dev_scale=scale_d.ptr)
    np.testing.assert_array_equal(out_d.get()[offset:], want)
    for d in (src_d, out_d, scale_d):
        d.free()
    rt.free(stats)
