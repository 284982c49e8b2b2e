"""`cpu`: NumPy restatement of the reference CPU transformer.  ORACLE ONLY.

Test infrastructure: registers a transformer named "cpu" that evaluates an op
graph one op at a time with the NumPy call
ngraph/transformers/cputransform.py:512-761 generates for it (table in
oracle/numpy_ops.py), on float32 buffers (cputransform.py:998-1007), after the
SimplePrune rewrite the CPU transformer also runs (cputransform.py:905-917; restated in
oracle/prune.py).
It shares the graph front (axes, views, ordering) with the product so the same
graph can be run on both; what pins that shared front are the NumPy
expressions written out in the tests themselves, as in the reference's own
tests.  Nothing in the product imports this module.
"""
from __future__ import division

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.transformers.base import (ComputationGraphTransformer, DeviceBufferStorage,
                                          DeviceTensor)
from oracle import numpy_ops
from oracle.prune import OraclePrune

# Graph op class -> name of its NumPy call in oracle/numpy_ops.py, one row per `generate_op`
# overload of ngraph/transformers/cputransform.py:512-761 (looked up along the op's class
# hierarchy, so a subclass of a listed op takes its parent's row).
NUMPY_CALL_OF = {
    "AbsoluteOp": "abs", "CosOp": "cos", "ExpOp": "exp", "LogOp": "log", "NegativeOp": "neg",
    "ReciprocalOp": "rcp", "SignOp": "sgn", "SinOp": "sin", "SqrtOp": "sqrt", "SquareOp": "sqr",
    "TanhOp": "tanh", "SigmoidAtomicOp": "sig",
    "Add": "add", "Subtract": "sub", "Multiply": "mul", "Divide": "div",
    "FloorDivide": "int_div", "Mod": "mod", "Power": "pow", "Maximum": "maximum",
    "Minimum": "minimum", "Equal": "eq", "NotEqual": "ne", "Less": "lt", "LessEqual": "le",
    "Greater": "gt", "GreaterEqual": "ge",
    "Sum": "sum", "Prod": "prod", "Max": "max", "Min": "min", "Argmax": "argmax",
    "Argmin": "argmin",
}


def numpy_call_name(op):
    for cls in type(op).__mro__:
        if cls.__name__ in NUMPY_CALL_OF:
            return NUMPY_CALL_OF[cls.__name__]
    return None


class NumpyDeviceBufferStorage(DeviceBufferStorage):
    def __init__(self, transformer, bytes, dtype, **kwargs):
        super(NumpyDeviceBufferStorage, self).__init__(transformer, bytes, dtype, **kwargs)
        np_dtype = dtype if isinstance(dtype, np.dtype) else np.dtype(np.float32)
        self.np_dtype = np_dtype
        self.data = np.zeros(max(int(bytes) // np_dtype.itemsize, 1), dtype=np_dtype)

    def create_device_tensor(self, tensor_description):
        return NumpyDeviceTensor(self.transformer, self, tensor_description)


class NumpyDeviceTensor(DeviceTensor):
    def transform_allocate(self):
        pass

    @property
    def view(self):
        """np.ndarray view of the buffer (cputransform.py:278-290)."""
        td = self.tensor_description
        base = self.device_buffer.data
        itemsize = base.dtype.itemsize
        return np.lib.stride_tricks.as_strided(
            base[td.offset:], shape=td.shape,
            strides=tuple(s * itemsize for s in td.full_strides), writeable=True)

    def get(self, tensor):
        value = np.array(self.view, copy=True)
        if tensor is None:
            return value
        tensor[...] = value
        return tensor

    def __getitem__(self, key):
        return self.view[key]

    def __setitem__(self, key, value):
        self.view.__setitem__(key if key is not Ellipsis else (), value)


class NumpyTransformer(ComputationGraphTransformer):
    transformer_name = "cpu"
    default_rtol = 1e-05
    default_atol = 1e-08

    def __init__(self, **kwargs):
        super(NumpyTransformer, self).__init__(**kwargs)
        self.graph_passes = [OraclePrune()]

    def device_buffer_storage(self, bytes, dtype, name):
        return NumpyDeviceBufferStorage(self, bytes, dtype, name="a_" + name)

    def start_transform_allocate(self):
        pass

    def finish_transform_allocate(self):
        pass

    def finish_transform(self):
        pass

    def allocate_storage(self):
        pass

    def _view(self, op):
        return self.get_tensor_description_tensor_view(op.forwarded.tensor_description()).view

    def transform_ordered_ops(self, computation, ordered_ops, name):
        steps = []
        for op in ordered_ops:
            op = op.forwarded
            if not op.is_device_op:
                continue
            steps.append(self._step(op))

        def run():
            for step in steps:
                step()
        computation.executor = run
        return name

    def _step(self, op):
        view = self._view
        name = numpy_call_name(op)
        if isinstance(op, og.AssignOp):
            return lambda: view(op.args[0]).__setitem__((), view(op.args[1]))      # :723-725
        if isinstance(op, og.Fill):
            return lambda: view(op.args[0]).fill(op.scalar)                        # :646-648
        if isinstance(op, og.TensorSizeOp):
            return lambda: view(op).fill(op.reduction_axes.size)                   # :759-761
        if isinstance(op, og.ContiguousOp):
            return lambda: view(op).__setitem__((), view(op.args[0]))
        if isinstance(op, og.OneHotOp):
            def onehot():                                                          # :702-704
                o, x = view(op), view(op.args[0])
                o[:] = np.eye(o.shape[0])[:, x.astype(np.int32)]
            return onehot
        if isinstance(op, og.RngOp):
            def fill_random():                                       # cputransform.py:580-587
                out = view(op)
                if op.distribution == "uniform":
                    out[()] = np.random.uniform(low=op.params["low"], high=op.params["high"], size=out.shape)
                else:
                    out[()] = np.random.normal(loc=op.params["loc"], scale=op.params["scale"], size=out.shape)
            return fill_random
        if isinstance(op, og.LookupTableOp):
            def lookup():                                            # cpuengine.py:421-422 fprop_lut
                view(op)[:] = view(op.args[0]).take(view(op.args[1]).astype(int), op.lut_axis)
            return lookup
        if isinstance(op, og.ReductionOp):
            x_axes = op.args[0].forwarded.axes
            np_axis = tuple(x_axes.index(a) for a in op.reduction_axes)           # :348-370
            np_axis = np_axis[0] if len(np_axis) == 1 else np_axis

            def reduce():
                x, out = view(op.args[0]), view(op)
                if np_axis == ():
                    out[()] = 0 if name in ("argmax", "argmin") else x
                elif name in ("argmax", "argmin"):
                    if isinstance(np_axis, tuple):
                        raise NotImplementedError("argmax over several axes")
                    out[()] = getattr(np.ndarray, name)(x, axis=np_axis)
                else:
                    with np.errstate(all="ignore"):
                        numpy_ops.REDUCE[name](x, axis=np_axis, out=out)
            return reduce
        if name == "sig":
            return lambda: view(op).__setitem__((), numpy_ops.unary("sig", view(op.args[0])))
        if name in numpy_ops.UNARY:
            fn = numpy_ops.UNARY[name]

            def unary():
                with np.errstate(all="ignore"):
                    fn(view(op.args[0]), out=view(op))
            return unary
        if name in numpy_ops.BINARY:
            fn = numpy_ops.BINARY[name]

            def binary():
                with np.errstate(all="ignore"):
                    fn(view(op.args[0]), view(op.args[1]), out=view(op))
            return binary
        raise ValueError("cpu oracle has no rule for op {}".format(op))
