"""oracle/prune.py (the oracle's own restatement of the reference's SimplePrune,
ngraph/transformers/passes/passes.py:499-628) pinned rule by rule: the reference's own test of
the pass (tests/test_graph_pass.py:22-39) and, for every rule, the graph it must leave and the
value that graph evaluates to, written as a NumPy expression here."""
import numpy as np
import pytest

import ngraph_hip as ng
from ngraph_hip.op_graph import op_graph as og
from oracle.prune import OraclePrune
from oracle.cpu_transformer import NumpyTransformer


def _pruned(op):
    OraclePrune().wrapped_do_pass(ops=[op])
    return op.forwarded


def _name(op):
    return type(op).__name__


def _reads(op, tensor):
    """Is `op` the placeholder `tensor` itself or a read of it?"""
    return op is tensor or getattr(op, "tensor", None) is tensor


def test_log_of_exp_of_a_constant_forwards_to_the_constant():
    # tests/test_graph_pass.py:22-39 of the reference
    base = og.as_op(ng.constant(5.0))
    graph = ng.log(ng.exp(base))
    OraclePrune().wrapped_do_pass(ops=[graph])
    assert graph.forwarded is base


def _axes():
    return ng.make_axes([ng.make_axis(3, name="A"), ng.make_axis(4, name="B")])


def test_multiplication_by_a_scalar_constant():
    x = ng.placeholder(_axes())
    assert _reads(_pruned(x * 1), x)
    assert _reads(_pruned(1 * x), x)
    minus = _pruned(x * -1)
    assert _name(minus) == "NegativeOp" and _reads(minus.args[0].forwarded, x)
    zero = _pruned(0 * x)
    assert zero.is_constant and float(np.asarray(_strip(zero).const)) == 0.0
    # any other factor stays a multiplication
    assert _name(_pruned(x * 2)) == "Multiply"


def _strip(op):
    """The scalar constant under the broadcast a replacement is given to fit the op's axes."""
    while not hasattr(op, "const") or op.const is None:
        op = op.args[0].forwarded
    return op


def test_addition_of_zero_and_negation_of_a_constant():
    x = ng.placeholder(_axes())
    assert _reads(_pruned(x + 0), x)
    assert _reads(_pruned(0 + x), x)
    assert _name(_pruned(x + 3)) == "Add"
    c = _pruned(ng.negative(ng.constant(2.5)))
    assert c.is_constant and float(np.asarray(_strip(c).const)) == -2.5


def test_sum_and_product_of_a_constant_count_the_reduced_elements():
    A, B = _axes()
    filled = ng.broadcast(ng.constant(1.5), [A, B])
    s = _pruned(ng.sum(filled, reduction_axes=[A]))
    assert s.is_constant and float(np.asarray(_strip(s).const)) == 1.5 * 3      # not 1.5 * 4, not 1.5 ** 3
    p = _pruned(ng.prod(filled, reduction_axes=[B]))
    assert p.is_constant and float(np.asarray(_strip(p).const)) == 1.5 ** 4


def test_log_of_a_quotient_of_an_exponential():
    x, d = ng.placeholder(_axes()), ng.placeholder(_axes())
    out = _pruned(ng.log(ng.exp(x) / d))
    # x - log(d): the subtraction's operands in this order
    assert _name(out) == "Subtract"
    assert _reads(out.args[0].forwarded, x)
    assert _name(out.args[1].forwarded) == "LogOp" and _reads(out.args[1].forwarded.args[0].forwarded, d)
    assert _reads(_pruned(ng.log(ng.exp(x))), x)
    assert _name(_pruned(ng.log(x / d))) == "LogOp"


@pytest.mark.parametrize("seed", [0, 1])
def test_the_pruned_graph_evaluates_to_the_unpruned_mathematics(seed):
    rs = np.random.RandomState(seed)
    A, B = _axes()
    x, d = ng.placeholder([A, B]), ng.placeholder([A, B])
    xv = rs.uniform(-2, 2, (3, 4)).astype(np.float32)
    dv = rs.uniform(0.5, 2, (3, 4)).astype(np.float32)
    graph = (ng.log(ng.exp(x) / d) + 0) * 1 + ng.sum(ng.broadcast(ng.constant(0.25), [A, B]), out_axes=[B]) \
        + (x * -1) * ng.prod(ng.broadcast(ng.constant(2.0), [A, B]), out_axes=[B])
    t = NumpyTransformer()
    try:
        got = np.array(t.computation(graph, x, d)(xv, dv))
    finally:
        t.close()
    x64, d64 = xv.astype(np.float64), dv.astype(np.float64)
    want = (x64 - np.log(d64)) + 0.25 * 3 + (-x64) * 2.0 ** 3
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
