"""Templates for the flex known-answer tests (ngraph/testing/flex_util.py:23-155)."""
from __future__ import print_function
import numpy as np

import ngraph_hip as ng
from ngraph_hip.testing.execution import executor
from ngraph_hip.testing.error_check import assert_allclose

MINIMUM_FLEX_VALUE = -2 ** 15
MAXIMUM_FLEX_VALUE = 2 ** 15 - 1


def get_placeholder_from_operand(operand, axes=None):
    if not isinstance(axes, ng.Axes):
        if not isinstance(operand, np.ndarray):
            axes = ()
        else:
            if len(operand.shape) > 1:
                rows, columns = operand.shape
                axes = ng.make_axes([ng.make_axis(length=rows), ng.make_axis(length=columns)])
            else:
                axes = ng.make_axes([ng.make_axis(length=operand.size)])
    return ng.placeholder(axes), axes


def execute_calculation(operands, first_operand, const_executor):
    """operands: [(in0[, in1], expected)]; one step -> exact equality, several -> flex tolerance."""
    iterations = len(operands) != 1
    results = []
    for step in operands:
        _operands, expected_result = step[:-1], step[-1]
        flex_result = const_executor(*_operands)
        results.append(flex_result)
        if iterations:
            assert_allclose(flex_result, expected_result)
        elif not isinstance(first_operand, np.ndarray):
            assert flex_result == expected_result, (flex_result, expected_result)
        else:
            assert np.array_equal(flex_result, expected_result), (flex_result, expected_result)
    return results


def template_one_placeholder(operands, ng_fun):
    first_operand = operands[0][0]
    ng_placeholder, _ = get_placeholder_from_operand(first_operand)
    with executor(ng_fun(ng_placeholder), ng_placeholder) as const_executor:
        return execute_calculation(operands, first_operand, const_executor)


def template_two_placeholders(operands, ng_fun):
    first_operand, second_operand = operands[0][0], operands[0][1]
    ng_placeholder1, axes = get_placeholder_from_operand(first_operand)
    ng_placeholder2, _ = get_placeholder_from_operand(second_operand, axes=axes)
    with executor(ng_fun(ng_placeholder1, ng_placeholder2),
                  ng_placeholder1, ng_placeholder2) as const_executor:
        return execute_calculation(operands, first_operand, const_executor)
