"""The five benchmark configurations at graph level.

`test_oracle_*` (CPU) pin oracle/configs.py against independent float64
restatements of the references the upstream tests hold: BatchNormReference
(frontends/neon/tests/test_batchnorm_layer.py:35-58), AdamReference
(test_optimizer.py:103-135, equal up to where epsilon enters) and the textbook
LSTM cell equations of lstm_ref.py.  The backend tests then run the ng graphs
built from the neon formulas on the oracle transformer ("cpu") and on
"hipgpu" and compare with oracle/configs.py on the same seeded inputs.
"""
import numpy as np
import pytest
from conftest import default_kernel_choice

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from oracle import configs
import oracle.cpu_transformer  # noqa: F401

RTOL, ATOL = 1e-5, 1e-6
BACKENDS = ["cpu", pytest.param("hipgpu", marks=pytest.mark.gpu),
            pytest.param("hipgpu-nofuse", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def transformer(request):
    if request.param == "hipgpu-nofuse":
        t = ngt.make_transformer_factory("hipgpu", fusion=False)()
    else:
        t = ngt.make_transformer_factory(request.param)()
    yield t
    t.close()


# ------------------------------------------------------------------ oracle pins (CPU)
def test_oracle_c1_against_float64():
    x, a, b = configs.c1_inputs((64, 257))
    want = np.tanh(np.float64(a) * x.astype(np.float64) + np.float64(b)) / (1 + np.exp(-x.astype(np.float64)))
    np.testing.assert_allclose(configs.c1_cpu(x, a, b), want, rtol=2e-6, atol=1e-7)


def test_oracle_c2_against_batchnorm_reference():
    x, gamma, beta = configs.c2_inputs(8, 3000)
    x64 = x.astype(np.float64)
    xmean = x64.mean(axis=1, keepdims=True)
    xvar = x64.var(axis=1, keepdims=True)
    want = gamma[:, None] * ((x64 - xmean) / np.sqrt(xvar + 1e-5)) + beta[:, None]
    y, mean, var = configs.c2_cpu(x, gamma, beta)
    np.testing.assert_allclose(mean, xmean.squeeze(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var, xvar.squeeze(), rtol=1e-5)
    np.testing.assert_allclose(y, want, rtol=1e-4, atol=1e-5)


def test_oracle_c3_against_adam_reference():
    p, g, m, v = configs.c3_inputs(5000)
    p64, g64 = p.astype(np.float64), g.astype(np.float64)
    m64, v64 = np.zeros_like(p64), np.zeros_like(p64)
    lr, b1, b2, eps = 1e-3, 0.9, 0.999, 1e-8
    for t in (1, 2, 3):
        configs.c3_cpu(p, g, m, v, t)
        m64 = b1 * m64 + (1 - b1) * g64
        v64 = b2 * v64 + (1 - b2) * g64 * g64
        ell = lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)
        p64 = p64 - ell * m64 / (np.sqrt(v64) + eps)       # optimizer.py:457-468 form
        m_hat, v_hat = m64 / (1 - b1 ** t), v64 / (1 - b2 ** t)
        # AdamReference form differs only in where epsilon enters
        big = np.abs(g64) > 1e-4          # where epsilon is negligible the two forms agree
        alt = ell * m64 / (np.sqrt(v64) + eps) - lr * m_hat / (np.sqrt(v_hat) + eps)
        assert np.abs(alt[big]).max() < 1e-5     # the upstream test tolerance
    np.testing.assert_allclose(m, m64, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(v, v64, rtol=1e-5, atol=1e-12)
    np.testing.assert_allclose(p, p64, rtol=1e-5, atol=1e-6)


def test_oracle_c4_against_textbook_lstm():
    gates, cprev = configs.c4_inputs(32, 6)
    g64, c64 = gates.astype(np.float64).T, cprev.astype(np.float64).T     # logical [4H,N], [H,N]
    H = 32
    sig = lambda z: 1 / (1 + np.exp(-z))
    i, f, o, g = sig(g64[:H]), sig(g64[H:2 * H]), sig(g64[2 * H:3 * H]), np.tanh(g64[3 * H:])
    c_want = f * c64 + i * g
    h_want = o * np.tanh(c_want)
    c, h, db = configs.c4_cpu(gates, cprev)
    np.testing.assert_allclose(c, c_want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(h, h_want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(db, g64.sum(axis=1), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------ graphs on the backends
@pytest.mark.parametrize("shape", [(1024, 1024), (33, 65)])
def test_c1_graph(transformer, shape):
    x_np, a, b = configs.c1_inputs(shape)
    H, W = ng.make_axis(shape[0], name="H"), ng.make_axis(shape[1], name="W")
    x, pa, pb = ng.placeholder([H, W]), ng.placeholder(()), ng.placeholder(())
    f = transformer.computation(ng.tanh(pa * x + pb) * ng.sigmoid(x), x, pa, pb)
    np.testing.assert_allclose(f(x_np, a, b), configs.c1_cpu(x_np, a, b), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dims", [(16, 7, 7, 8), (256, 14, 14, 4), (5, 3, 3, 2)])
def test_c2_graph(transformer, dims):
    Cn, Hn, Wn, Nn = dims
    x_np, gamma_np, beta_np = configs.c2_inputs(Cn, Hn * Wn * Nn)
    y_w, mean_w, var_w = configs.c2_cpu(x_np, gamma_np, beta_np)
    C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", dims))
    x = ng.placeholder([C, H, W, N])
    gamma = ng.variable([C], initial_value=gamma_np)
    beta = ng.variable([C], initial_value=beta_np)
    y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    f = transformer.computation([y, xmean, xvar], x)
    y_g, mean_g, var_g = f(x_np.reshape(dims))
    np.testing.assert_allclose(mean_g, mean_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(var_g, var_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y_g.reshape(Cn, -1), y_w, rtol=RTOL, atol=1e-5)


@pytest.mark.parametrize("n", [1 << 16, 1000003])
def test_c3_graph(transformer, n):
    p_np, g_np, m_np, v_np = configs.c3_inputs(n)
    P = ng.make_axis(n, name="P")
    p = ng.variable([P], initial_value=p_np)
    grad = ng.placeholder([P])
    opt = neon.Adam()
    opt()
    updates, m, v = opt.variable_update(p, grad)
    f = transformer.computation([updates, ng.value_of(m), ng.value_of(v)] if False else updates, grad)
    read = transformer.computation([p * 1.0, m * 1.0, v * 1.0])
    for t in (1, 2):
        configs.c3_cpu(p_np, g_np, m_np, v_np, t)
        f(g_np)
    p_g, m_g, v_g = read()
    np.testing.assert_allclose(m_g, m_np, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(v_g, v_np, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(p_g, p_np, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Hn,Nn", [(1024, 64), (48, 5)])
def test_c4_graph(transformer, Hn, Nn):
    gates_np, cprev_np = configs.c4_inputs(Hn, Nn)
    c_w, h_w, db_w = configs.c4_cpu(gates_np, cprev_np)
    H, N, G = ng.make_axis(Hn, name="H"), ng.make_axis(Nn, name="N"), ng.make_axis(4 * Hn, name="G")
    # storage is the transpose: placeholders hold [N, 4H] / [N, H]; the graph works on [.., N] views
    gates_st = ng.placeholder([N, G])
    cprev_st = ng.placeholder([N, H])
    gates = ng.axes_with_order(gates_st, [G, N])
    c_prev = ng.axes_with_order(cprev_st, [H, N])
    parts = {k: ng.cast_axes(ng.tensor_slice(gates, [slice(j * Hn, (j + 1) * Hn), slice(None)]), [H, N])
             for j, k in enumerate(("i", "f", "o", "g"))}
    h, c = neon.lstm_cell(parts, c_prev, H, None)
    db = ng.sum(gates, out_axes=[G])
    f = transformer.computation([c, h, db], gates_st, cprev_st)
    c_g, h_g, db_g = f(gates_np, cprev_np)
    np.testing.assert_allclose(c_g, c_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(h_g, h_w, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(db_g, db_w, rtol=RTOL, atol=1e-5)
    group = getattr(transformer, "kernel_groups", {}).get(f)
    if group is not None and getattr(transformer, "fusion", False) and default_kernel_choice() and Hn * Nn >= 4096:
        # the cell and the bias gradient's column sum went to the device as ONE launch
        assert group._pairs == {0}, (group._pairs, [type(k).__name__ for k in group.kernels])


@pytest.mark.gpu
@pytest.mark.parametrize("policy", [0, 1, 2, 3])
def test_cache_policy_does_not_change_results(policy, monkeypatch):
    """Non-temporal loads / stores are a cache hint only: forcing each of the four variants
    of the pre-built Adam and batch-norm kernels gives bit-identical results."""
    check_names = default_kernel_choice()        # before this test sets a knob itself

    def adam_and_bn():
        out = []
        t = ngt.make_transformer_factory("hipgpu")()
        n = 100000
        p_np, g_np, _, _ = configs.c3_inputs(n)
        P = ng.make_axis(n, name="P")
        p, grad = ng.variable([P], initial_value=p_np), ng.placeholder([P])
        opt = neon.Adam()
        opt()
        updates, m, v = opt.variable_update(p, grad)
        f = t.computation(updates, grad)
        read = t.computation([p * 1.0, m * 1.0, v * 1.0])
        f(g_np)
        f(g_np)
        out.extend(np.array(a) for a in read())
        assert not check_names or \
            any("special:adam" in d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds)
        t.close()
        t = ngt.make_transformer_factory("hipgpu")()
        dims = (64, 16, 16, 16)
        x_np, gamma_np, beta_np = configs.c2_inputs(dims[0], dims[1] * dims[2] * dims[3])
        C, H, W, N = (ng.make_axis(k, name=s) for s, k in zip("CHWN", dims))
        x = ng.placeholder([C, H, W, N])
        gamma, beta = ng.variable([C], initial_value=gamma_np), ng.variable([C], initial_value=beta_np)
        y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
        f = t.computation([y, xmean, xvar], x)
        out.extend(np.array(a) for a in f(x_np.reshape(dims)))
        assert not check_names or \
            any("special:batchnorm" in d or "/chain-of-" in d     # (rows this short merge into a row chain once one is compiled)
                for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds)
        t.close()
        return out

    monkeypatch.setenv("NGH_CACHE_POLICY", "0")
    want = adam_and_bn()
    monkeypatch.setenv("NGH_CACHE_POLICY", str(policy))
    got = adam_and_bn()
    for a, b in zip(got, want):
        np.testing.assert_array_equal(a, b)


# ------------------------------------------------------------------ other learning rules
def _run_rule(transformer, make_updates, n, steps=3):
    rs = np.random.RandomState(n)
    p0 = rs.normal(0, 0.1, n).astype(np.float32)
    grads = [rs.normal(0, 0.01, n).astype(np.float32) for _ in range(steps)]
    P = ng.make_axis(n, name="P")
    p, grad = ng.variable([P], initial_value=p0), ng.placeholder([P])
    updates = make_updates(p, grad)
    f = transformer.computation(updates, grad)
    read = transformer.computation(p * 1.0)
    for g in grads:
        f(g)
    return p0, grads, np.array(read())


@pytest.mark.parametrize("n", [1 << 16, 100003])
@pytest.mark.parametrize("nesterov", [False, True])
def test_sgd_momentum_with_kahan_update(transformer, n, nesterov):
    """optimizer.py:285-310 restated in float64 (the compensated sum makes fp32 track it)."""
    opt = neon.GradientDescentMomentum(0.1, momentum_coef=0.9, wdecay=0.01, nesterov=nesterov)
    p0, grads, got = _run_rule(transformer, lambda p, g: opt.variable_update(p, g)[0], n)
    p, vel = p0.astype(np.float64), np.zeros(n)
    for g in grads:
        lr = -0.1 * (g.astype(np.float64) + 0.01 * p)
        vel = vel * 0.9 + lr
        p = p + ((0.9 * vel + lr) if nesterov else vel)
    np.testing.assert_allclose(got, p, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("n", [1 << 16, 100003])
def test_rmsprop(transformer, n):
    opt = neon.RMSProp(decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6, wdecay=0.01, momentum_coef=0.5)
    p0, grads, got = _run_rule(transformer, lambda p, g: opt.variable_update(p, g)[0], n)
    p, state, vel = p0.astype(np.float64), np.ones(n), np.zeros(n)
    for g in grads:
        g = g.astype(np.float64)
        state = 0.95 * state + 0.05 * g * g
        vel = vel * 0.5 + 2e-3 * g / np.sqrt(state + 1e-6) + 2e-3 * 0.01 * p
        p = p - vel
    np.testing.assert_allclose(got, p, rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("n", [1 << 16, 100003])
def test_adagrad(transformer, n):
    opt = neon.Adagrad(learning_rate=0.01, epsilon=1e-6)
    p0, grads, got = _run_rule(transformer, lambda p, g: opt.variable_update(p, g)[0], n)
    p, state = p0.astype(np.float64), np.zeros(n)
    for g in grads:
        g = g.astype(np.float64)
        state = state + g * g
        p = p - 0.01 * g / np.sqrt(state + 1e-6)
    np.testing.assert_allclose(got, p, rtol=2e-5, atol=1e-6)
