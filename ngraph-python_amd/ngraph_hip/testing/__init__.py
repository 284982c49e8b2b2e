from ngraph_hip.testing.execution import (executor, ExecutorFactory, is_flex_factory,  # noqa: F401
                                          numeric_derivative, check_derivative)
from ngraph_hip.testing.error_check import assert_allclose  # noqa: F401
from ngraph_hip.testing.random import RandomTensorGenerator  # noqa: F401
