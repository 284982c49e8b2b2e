"""Test harness: run graph ops through the current transformer factory.

Mirrors ngraph/testing/execution.py:28-168: `executor(results, *params)` is
a context manager yielding a callable; `ExecutorFactory` owns a transformer
made by `ngt.make_transformer()` and closes it on exit.
"""
from contextlib import contextmanager

import numpy as np

import ngraph_hip.transformers as ngt


class ExecutorFactory(object):
    def __init__(self):
        pass

    def __enter__(self):
        self.transformer = ngt.make_transformer()
        return self

    def __exit__(self, *args):
        self.transformer.close()

    def executor(self, results, *parameters):
        return self.transformer.computation(results, *parameters)

    def get_tensor_view_value(self, op, host_tensor=None):
        return self.transformer.get_tensor_view_value(op, host_tensor)

    def numeric_derivative(self, f, p_x, dx, *params):
        """df/dp_x by one-sided differences of size dx (execution.py:75-87, 170-216)."""
        comp = self.transformer.computation(f, p_x, *params)

        def helper(x, *args):
            return numeric_derivative(lambda xx: comp(xx, *args), x, dx)
        return helper

    def derivative(self, f, px, *parameters):
        """The full derivative of f with respect to placeholder px, indexed (f..., px...): one
        backward evaluation per element of f, each with a one-hot error (execution.py:89-138)."""
        import ngraph_hip as ng
        fshape, xshape = f.axes.lengths, px.axes.lengths
        if len(fshape) == 0:
            return self.transformer.computation(ng.deriv(f, px), px, *parameters)
        initial_adjoint = ng.placeholder(f.axes).named("adj")
        comp = self.transformer.computation(ng.deriv(f, px, error=initial_adjoint), initial_adjoint, px,
                                            *parameters)

        def helper(x, *args):
            adjoint = np.zeros(fshape, dtype=np.float32)
            out = np.empty(tuple(fshape) + tuple(xshape), dtype=np.float32)
            for index in np.ndindex(*fshape):
                adjoint[index] = 1
                out[index] = comp(adjoint, x, *args)
                adjoint[index] = 0
            return out
        return helper


@contextmanager
def executor(results, *parameters):
    with ExecutorFactory() as ex:
        yield ex.executor(results, *parameters)


def numeric_derivative(f, x, dx):
    """df/dx at x numerically, indexed (f..., x...).  Not for min/max at ties."""
    x = np.array(x, dtype=np.float32)
    y = np.copy(f(x))
    d = np.zeros(tuple(np.shape(y)) + x.shape, dtype=np.float32)
    for index in np.ndindex(*x.shape):
        old = x[index]
        x[index] = old + dx
        d[(Ellipsis,) + index] = (f(x) - y) / dx
        x[index] = old
    return d


def check_derivative(f, x, delta, x_value, parameters=(), parameter_values=(), **kwargs):
    """Numeric against symbolic derivative of f with respect to x at x_value
    (execution.py:218-243)."""
    with ExecutorFactory() as ex:
        numeric = ex.numeric_derivative(f, x, delta, *parameters)
        symbolic = ex.derivative(f, x, *parameters)
        np.testing.assert_allclose(numeric(x_value, *parameter_values), symbolic(x_value, *parameter_values),
                                   **kwargs)


def is_flex_factory(factory=None):
    name = getattr(factory, "name", "") if factory is not None else ""
    return "flex" in name
