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
from ngraph_hip.runtime.programs import stage_programs, render  # noqa: E402

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


def pattern_softmax_rows(t):
    N, C = _axes(N=4096, C=1000)
    x = ng.placeholder([N, C])
    return t.computation(ng.softmax(x, normalization_axes=ng.make_axes([C])), x)


def pattern_log_softmax_rows(t):
    N, C = _axes(N=4096, C=1000)
    x = ng.placeholder([N, C])
    shifted = x - ng.max(x, out_axes=[N])
    return t.computation(shifted - ng.log(ng.sum(ng.exp(shifted), out_axes=[N])), x)


def pattern_batchnorm_short_rows(t):
    # (the same statements as pattern_batchnorm: with rows of up to 8192 elements the statistics
    # and the normalise kernel merge into one row chain that also writes the statistics out)
    return pattern_batchnorm(t)


def _layer_norm_pattern(affine):
    def build(t):
        N, C = _axes(N=4096, C=1000)
        x = ng.placeholder([N, C])
        mean, var = ng.mean(x, out_axes=[N]), ng.variance(x, out_axes=[N])
        y = (x - mean) * ng.reciprocal(ng.sqrt(var + 1e-5))
        if affine:
            g, b = ng.placeholder([C]), ng.placeholder([C])
            return t.computation(g * y + b, x, g, b)
        return t.computation(y, x)
    return build


# patterns whose kernels merge into one row chain (rows of up to 8192 elements along the
# contiguous axis): the chain is built in, so that these run as one launch without run-time
# compilation, whatever their size
CHAINS = ("softmax_rows", "log_softmax_rows", "batchnorm_short_rows", "layer_norm_rows", "layer_norm_affine_rows")

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
    ("softmax_rows", "hipgpu", pattern_softmax_rows),
    ("log_softmax_rows", "hipgpu", pattern_log_softmax_rows),
    ("batchnorm_short_rows", "hipgpu", pattern_batchnorm_short_rows),
    ("layer_norm_rows", "hipgpu", _layer_norm_pattern(False)),
    ("layer_norm_affine_rows", "hipgpu", _layer_norm_pattern(True)),
]


def collect():
    """Program records for every stage of every pattern that a compiled kernel can run."""
    programs, seen = [], set()
    for name, backend, build in PATTERNS:
        if backend not in ngt.transformer_choices():
            continue
        t = ngt.make_transformer_factory(backend, dry_run=True)()
        # (the patterns stand for tensors of any size: their kernels stay separate programs here,
        # whether or not the small stand-ins would merge into a row chain)
        t.chain_kernels = name in CHAINS
        f = build(t)
        t.initialize()
        kernels = t.kernel_groups[f].kernels
        for kernel in kernels:
            kernel.bind_buffers()
        programs += stage_programs(kernels, name, seen, vector_only=True)
        t.close()
    return programs


# programs that one launch runs side by side: the LSTM cell and the column sum for its bias gradient
PAIRS = [("lstm_cell_k0", "sum_across_small_k0")]

HEADER = ["// GENERATED by gen_programs.py from the host lowering -- do not edit.",
          "// One entry per streaming elementwise op program that gets a pre-built kernel."]


if __name__ == "__main__":
    text = render(collect(), HEADER, pairs=PAIRS)
    if "--check" in sys.argv:
        sys.exit(0 if open(OUT).read() == text else 1)
    with open(OUT, "w") as fh:
        fh.write(text)
    print("wrote", OUT)
