"""Runner for the flex known-answer vectors of tests/golden/flex_vectors.json.

A vector is an op and a sequence of steps (operands..., expected result) applied to ONE
computation, so that the exponents a step leaves behind are what the next step meets.  The
acceptance rule is the reference's (ngraph/testing/flex_util.py:114-135): a single step must
reproduce its result exactly -- the flex rounding is fully determined -- while a sequence is
compared with the transformer's flex tolerance, because the reference recorded those with its
own exponent history.
"""
import numpy as np

import ngraph_hip as ng
from ngraph_hip.testing.execution import executor
from ngraph_hip.testing.error_check import assert_allclose


def placeholders_like(operands):
    """One placeholder per operand; array operands of equal shape share their axes, scalars
    have none."""
    by_shape, made = {}, []
    for value in operands:
        shape = np.shape(value) if isinstance(value, np.ndarray) else ()
        if shape not in by_shape:
            by_shape[shape] = ng.make_axes([ng.make_axis(length=n) for n in shape])
        made.append(ng.placeholder(by_shape[shape]))
    return made


def check_steps(run, steps):
    """Feed every step's operands to `run` (the computation) and compare with its expected value."""
    exact = len(steps) == 1
    for step in steps:
        operands, want = step[:-1], step[-1]
        got = run(*operands)
        if not exact:
            assert_allclose(got, want)
        elif isinstance(operands[0], np.ndarray):
            assert np.array_equal(got, want), (got, want)
        else:
            assert got == want, (got, want)


def run_vector(op, steps):
    """Build op(placeholders) once, then run the steps through it."""
    inputs = placeholders_like(steps[0][:-1])
    with executor(op(*inputs), *inputs) as run:
        check_steps(run, steps)
