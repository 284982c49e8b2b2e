"""ngraph_hip: an MI355X-native backend for ngraph-python's fused
elementwise / reduction / flex16 path, with the slice of the `ngraph` API that
path is driven through (`import ngraph_hip as ng`).

    import ngraph_hip as ng
    import ngraph_hip.transformers as ngt

    x = ng.placeholder(ng.make_axes([ng.make_axis(1024, name="H"), ng.make_axis(64, name="N")]))
    with ngt.make_transformer_factory("hipgpu")() as t: ...
"""
from ngraph_hip.op_graph.axes import (  # noqa: F401
    Axis, Axes, FlattenedAxis, TensorDescription, make_axis, make_axes, default_dtype,
    default_int_dtype)
from ngraph_hip.op_graph.op_graph import (  # noqa: F401
    Op, TensorOp, AssignableTensorOp, AssignOp, SequentialOp, ComputationOp, TensorValueOp,
    absolute, add, argmax, argmin, as_op, as_ops, assign, axes_with_order, batch_size, broadcast,
    cast_axes, cast_role, computation, constant, cos, divide, doall, equal, exp, expand_dims, fill,
    flatten, flatten_at, floordivide, greater, greater_equal, less, less_equal, log, max, maximum,
    mean, min, minimum, mod, multiply, negative, not_equal, one_hot, lookuptable, uniform, normal,
    persistent_tensor,
    placeholder, power, prod, reciprocal, safelog, sequential, sigmoid, sigmoidAtomic, sign, sin,
    slice_along_axis, softmax, sqrt, square, squared_L2, subtract, sum, tanh, temporary,
    tensor_size, tensor_slice, unflatten, value_of, variable, variance, Transpose,
    cross_entropy_multi, cross_entropy_binary, cross_entropy_binary_inner, UnmatchedAxesError,
    stack, concat_along_axis)
from ngraph_hip.op_graph.op_graph import ContiguousOp as _ContiguousOp
from ngraph_hip.op_graph.autodiff import deriv  # noqa: F401


def contiguous(x):
    """A C-contiguous copy of x (a device copy)."""
    return _ContiguousOp(x)


__version__ = "0.1.0"
