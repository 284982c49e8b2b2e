"""Test harness: run graph ops through the current transformer factory.

Mirrors ngraph/testing/execution.py:28-168: `executor(results, *params)` is
a context manager yielding a callable; `ExecutorFactory` owns a transformer
made by `ngt.make_transformer()` and closes it on exit.
"""
from contextlib import contextmanager

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


@contextmanager
def executor(results, *parameters):
    with ExecutorFactory() as ex:
        yield ex.executor(results, *parameters)


def is_flex_factory(factory=None):
    name = getattr(factory, "name", "") if factory is not None else ""
    return "flex" in name
