"""Activations, costs and dropout of the neon front: elementwise composites on the fused path.

Inputs and reference formulas follow ngraph/frontends/neon/tests/test_activations.py:64-170,
test_costs.py:27-91 and test_dropout.py:31-85 (forward values; derivatives are covered by
tests/test_autodiff.py).
"""
import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from ngraph_hip.testing import executor
import oracle.cpu_transformer  # noqa: F401

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


ACTIVATIONS = [
    ("Identity", neon.Identity(), lambda x: x, 0.0),
    ("Rectlin", neon.Rectlin(), lambda x: np.maximum(x, 0), 0.0),
    ("LeakyRectlin", neon.Rectlin(slope=0.2), lambda x: np.maximum(x, 0) + np.minimum(x, 0) * np.float32(0.2), 1e-7),
    ("RectlinClip", neon.Rectlinclip(cutoff=0.2), lambda x: np.minimum(np.maximum(x, 0), np.float32(0.2)), 0.0),
    ("Explin", neon.Explin(alpha=0.5), lambda x: np.maximum(x, 0) + 0.5 * (np.exp(np.minimum(x, 0.0)) - 1), 1e-6),
    ("Normalizer", neon.Normalizer(divisor=128.), lambda x: x / 128.0, 0.0),
    ("Tanh", neon.Tanh(), lambda x: np.tanh(x.astype(np.float64)), 2e-7),
    ("Logistic", neon.Logistic(), lambda x: 1.0 / (1.0 + np.exp(-x.astype(np.float64))), 2e-7),
    ("Softmax", neon.Softmax(), lambda x: np.exp(x - 1.0) / np.sum(np.exp(x - 1.0), axis=0, keepdims=True), 1e-6),
]
INPUTS = [np.array([[1], [3], [2]]), np.array([[0], [1], [-2]]), np.array([[4, 0], [-2, 5]]),
          np.array([[-1, -3], [-2, -4]])]


@pytest.mark.parametrize("x", INPUTS, ids=["all_positive_1d", "mixed_1d", "mixed_2d", "all_negative_2d"])
@pytest.mark.parametrize("name,act,ref,rtol", ACTIVATIONS, ids=[a[0] for a in ACTIVATIONS])
def test_activation(backend, name, act, ref, rtol, x):
    x = x.astype(np.float32)
    X = ng.placeholder([ng.make_axis(x.shape[0]), ng.make_axis(x.shape[1], name="N")])
    with executor(act(X), X) as f:
        np.testing.assert_allclose(f(x), ref(x), rtol=max(rtol, 1e-7), atol=1e-7)


def _safelog(x):
    # op_graph.py:3070-3072
    return np.maximum(np.log(x + np.exp(-50)), -50)


COSTS = [
    ("cross_entropy_multi", lambda Y, T: ng.cross_entropy_multi(Y, T),
     lambda y, t: np.sum(-t * _safelog(y), axis=0)),
    ("cross_entropy_binary", lambda Y, T: ng.cross_entropy_binary(Y, T),
     lambda y, t: np.sum(-t * _safelog(y) - (1 - t) * _safelog(1 - y))),
    ("sum_squared", neon.sum_squared, lambda y, t: np.sum((y - t) ** 2) / 2),
    ("mean_squared", neon.mean_squared, lambda y, t: np.mean((y - t) ** 2) / 2),
]


@pytest.mark.parametrize("y,t", [([0.5, 0.9, 0.1, 0.0001], [0.5, 0.99, 0.01, 0.2]),
                                 ([0.5, 1.0, 0.0, 0.0001], [0.5, 0.0, 1.0, 0.2])])
@pytest.mark.parametrize("name,build,ref", COSTS, ids=[c[0] for c in COSTS])
def test_costs(backend, name, build, ref, y, t):
    y, t = np.array(y, np.float32), np.array(t, np.float32)
    N = ng.make_axis(4)
    Y, T = ng.placeholder([N]), ng.placeholder([N])
    with executor(build(Y, T), Y, T) as f:
        np.testing.assert_allclose(f(y, t), ref(y.astype(np.float64), t.astype(np.float64)), rtol=2e-6)


@pytest.mark.parametrize("keep", [1.0, 0.75, 0.5])
def test_dropout_train(backend, keep):
    N, F = ng.make_axis(2, name="N"), ng.make_axis(32, name="F")
    inp = ng.placeholder([F, N])
    layer = neon.Dropout(keep=keep)
    out_op = layer(inp)
    x = np.random.RandomState(0).uniform(size=(32, 2)).astype(np.float32)
    with executor([out_op, layer.mask], inp) as f:
        out, mask = f(x)
        out1, mask1 = np.array(out).copy(), np.array(mask).copy()
        np.testing.assert_allclose(out1, x * mask1[:, None], rtol=1e-6)
        assert set(np.unique(mask1)) <= {0.0, 1.0}
        if keep == 1.0:
            assert mask1.all()
        else:
            out2, mask2 = f(x)
            assert (out1 != out2).any() and (mask1 != mask2).any()


def test_dropout_inference(backend):
    N, F = ng.make_axis(2, name="N"), ng.make_axis(32, name="F")
    inp = ng.placeholder([F, N])
    neon.Dropout.inference_mode = True
    try:
        out_op = neon.Dropout(keep=0.5)(inp)
    finally:
        neon.Dropout.inference_mode = False
    x = np.random.RandomState(1).uniform(size=(32, 2)).astype(np.float32)
    with executor(out_op, inp) as f:
        np.testing.assert_allclose(f(x), x * 0.5, rtol=1e-6)


# ---- optimizers driven by a cost (neon/tests/test_optimizer.py:139-330 compares with NumPy
# ---- reference classes; here the closed form is written out per rule) --------------------------
def _quadratic_problem():
    """cost_n = sum_f (w_f * x_fn - t_fn)^2 / 2: the gradient of the batch sum, divided by the
    batch size, is mean_n (w x - t) x."""
    F, N = ng.make_axis(5, name="F"), ng.make_axis(8, name="N")
    rs = np.random.RandomState(4)
    xv, tv = rs.normal(0, 1, (5, 8)).astype(np.float32), rs.normal(0, 1, (5, 8)).astype(np.float32)
    w0 = rs.normal(0, 0.5, 5).astype(np.float32)
    x, t = ng.placeholder([F, N]), ng.placeholder([F, N])
    w = ng.variable([F], initial_value=w0)
    cost = ng.sum(ng.square(w * x - t), out_axes=[N]) / 2

    def grad(wn):
        return ((wn[:, None] * xv - tv) * xv).mean(axis=1)
    return (x, t, w, cost), (xv, tv, w0.astype(np.float64)), grad


@pytest.mark.parametrize("rule", ["sgd", "sgd_momentum_clip", "rmsprop", "adagrad", "adam", "clip_norm"])
def test_optimizer_minimises_a_cost(backend, rule):
    (x, t, w, cost), (xv, tv, wn), grad = _quadratic_problem()
    steps = 4
    if rule == "sgd":
        opt = neon.GradientDescentMomentum(0.1)
        def ref(wn, state):
            return wn - 0.1 * grad(wn), state
    elif rule == "sgd_momentum_clip":
        opt = neon.GradientDescentMomentum(0.1, momentum_coef=0.9, gradient_clip_value=0.3, weight_clip_value=0.6)
        def ref(wn, state):
            vel = state.get("v", 0.0) * 0.9 - 0.1 * np.clip(grad(wn), -0.3, 0.3)
            return np.clip(wn + vel, -0.6, 0.6), {"v": vel}
    elif rule == "rmsprop":
        opt = neon.RMSProp(learning_rate=0.01)
        def ref(wn, state):
            g = grad(wn)
            s = 0.95 * state.get("s", 1.0) + 0.05 * g * g
            return wn - 0.01 * g / np.sqrt(s + 1e-6), {"s": s}
    elif rule == "adagrad":
        opt = neon.Adagrad(learning_rate=0.1)
        def ref(wn, state):
            g = grad(wn)
            s = state.get("s", 0.0) + g * g
            return wn - 0.1 * g / np.sqrt(s + 1e-6), {"s": s}
    elif rule == "adam":
        opt = neon.Adam(learning_rate=0.05)
        def ref(wn, state):
            g, k = grad(wn), state.get("k", 0) + 1
            m = 0.9 * state.get("m", 0.0) + 0.1 * g
            v = 0.999 * state.get("v", 0.0) + 0.001 * g * g
            ell = 0.05 * np.sqrt(1 - 0.999 ** k) / (1 - 0.9 ** k)
            return wn - ell * m / (np.sqrt(v) + 1e-8), {"k": k, "m": m, "v": v}
    else:
        opt = neon.GradientDescentMomentum(0.1, gradient_clip_norm=0.5)
        def ref(wn, state):
            g = grad(wn)
            return wn - 0.1 * g * (0.5 / max(np.sqrt((g * g).sum()), 0.5)), state
    train = opt.minimize(cost)
    read = w * 1.0
    t_ = ngt.make_transformer()
    try:
        f, r = t_.computation(train, x, t), t_.computation(read)
        state = {}
        for _ in range(steps):
            f(xv, tv)
            wn, state = ref(wn, state)
        np.testing.assert_allclose(r(), wn, rtol=2e-4, atol=2e-6)
    finally:
        t_.close()
