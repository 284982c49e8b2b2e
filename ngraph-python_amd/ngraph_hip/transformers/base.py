"""Transformer plugin interface: registry, factory, Computation, allocation flow.

Mirrors ngraph/transformers/base.py for what a backend plugs into:

* classes with a `transformer_name` register themselves in
  `Transformer.transformers` through the metaclass (base.py:265-279);
* `make_transformer_factory` / `set_transformer_factory` / `make_transformer`
  / `allocate_transformer` / `transformer_choices` (base.py:807-847);
* `Computation.__call__(*args)` or `(feed_dict=...)`: initialize -> copy
  parameters in -> executor() -> copy results out, returning an array, a
  tuple or a dict according to the shape of `returns` (base.py:94-136);
* `ComputationGraphTransformer`: run graph passes, one device buffer per
  base tensor, views per tensor description, then `transform_ordered_ops`
  per computation (base.py:478-801); adding a computation after the
  transformer is finalized raises ValueError (base.py:733-736).
"""
from __future__ import division
import abc
import weakref

import numpy as np

from ngraph_hip.op_graph.op_graph import Op, OrderedSet, computation as make_computation_op, \
    ComputationOp


class UnsupportedTransformerException(Exception):
    pass


class Computation(object):
    """A handle for a computation function."""

    _counter = 0

    def __init__(self, transformer, computation_op, **kwargs):
        self.transformer = transformer
        self.computation_op = computation_op
        self.computation_name = None
        self.executor = None
        self.name = "Computation_%d" % Computation._counter
        Computation._counter += 1

    def unpack_args_or_feed_dict(self, args, kwargs):
        feed_dict = kwargs.pop("feed_dict", None)
        if feed_dict is not None:
            if len(args) != 0:
                raise ValueError("Can not supply both positional and feed_dict arguments "
                                 "to Computation")
            args = tuple(feed_dict[param.tensor] for param in self.computation_op.parameters)
        if len(args) != len(self.computation_op.parameters):
            raise ValueError("Computation was expecting {expected} arguments, but was called "
                             "with {called}.".format(expected=len(self.computation_op.parameters),
                                                     called=len(args)))
        return args

    def __call__(self, *args, **kwargs):
        args = self.unpack_args_or_feed_dict(args, kwargs)
        self.transformer.initialize()
        self.transformer.host_to_device(self, self.computation_op.parameters, args)
        self.executor()

        def value(op):
            if op.is_tensor_op and "skip_returns" not in op.metadata:
                return self.transformer.device_to_host(self, op)
            return None

        cop = self.computation_op
        if cop.returns_kind == "op":
            return value(cop.returns)
        elif cop.returns_kind == "sequence":
            return tuple(value(op) for op in cop.returns)
        elif cop.returns_kind == "set":
            return dict((key, value(op)) for key, op in cop.returns_map.items())
        return None


class DeviceBufferStorage(object):
    """Something that can provide storage (base.py:140-210)."""

    def __init__(self, transformer, bytes, dtype, name=None, **kwargs):
        self.transformer = transformer
        self.bytes = bytes
        self.dtype = dtype
        self.name = name
        self.__views = dict()

    @property
    def views(self):
        return self.__views.values()

    def transform_allocate(self):
        self.transform_allocate_views()

    def transform_allocate_views(self):
        for view in self.views:
            view.transform_allocate()

    def device_tensor(self, tensor_description):
        tensor = self.__views.get(tensor_description.parameter_key, None)
        if tensor is not None:
            return tensor
        tensor = self.create_device_tensor(tensor_description)
        self.__views[tensor_description.parameter_key] = tensor
        return tensor

    def create_device_tensor(self, tensor_description):
        raise NotImplementedError


class DeviceTensor(object):
    """A handle to a tensor on the device (base.py:213-262)."""

    def __init__(self, transformer, device_buffer, tensor_description, name=None, **kwargs):
        self.transformer = transformer
        self.device_buffer = device_buffer
        self.tensor_description = tensor_description
        self.name = name

    @property
    def dtype(self):
        return self.tensor_description.dtype

    def transform_allocate(self):
        raise NotImplementedError

    def get(self, tensor):
        raise NotImplementedError

    def __getitem__(self, key):
        raise NotImplementedError

    def __setitem__(self, key, value):
        raise NotImplementedError


class Transformer_ABC_Meta(abc.ABCMeta):
    """Registers every subclass that names itself (base.py:265-279)."""

    def __init__(cls, name, bases, dict_):
        if not hasattr(cls, "transformers"):
            cls.transformers = {}
        transformer_name = getattr(cls, "transformer_name", None)
        if transformer_name is not None:
            cls.transformers[transformer_name] = cls
        super(Transformer_ABC_Meta, cls).__init__(name, bases, dict_)


class Transformer(object, metaclass=Transformer_ABC_Meta):
    """Produce an executable version of op-graphs (base.py:282-475)."""

    default_rtol = 1e-05
    default_atol = 1e-08

    def __init__(self, **kwargs):
        super(Transformer, self).__init__()
        self.graph_passes = []
        self.byte_alignment = 4

    def computation(self, results, *parameters):
        return self.add_computation(make_computation_op(results, *parameters))

    def add_computation(self, computation):
        return self.make_computation(computation)

    def make_computation(self, computation):
        return Computation(self, computation)

    def initialize(self):
        pass

    def register_graph_pass(self, graph_pass, position=None):
        if position is not None:
            self.graph_passes.insert(position, graph_pass)
        else:
            self.graph_passes.append(graph_pass)

    def set_output_statistics_file(self, statistics_file):
        pass

    def save_output_statistics_file(self):
        pass

    def close(self):
        pass

    @classmethod
    def get_default_tolerance(cls, desired):
        return cls.default_atol, cls.default_rtol

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ComputationGraphTransformer(Transformer):
    def __init__(self, **kwargs):
        super(ComputationGraphTransformer, self).__init__(**kwargs)
        self.computations = OrderedSet()
        self.device_buffers = None
        self.op_tensors = None
        self.op_tensor_views = None
        self.initialize_allocations()
        self.finalized = False
        self.allocated = False
        self.initialized = False
        self.ops = []

    def run_registered_graph_passes(self, ops, **kwargs):
        for graph_pass in self.graph_passes:
            graph_pass.wrapped_do_pass(ops=ops, **kwargs)
        return ops

    def initialize_allocations(self):
        self.op_tensors = dict()
        self.op_tensor_views = dict()
        self.device_buffers = OrderedSet()

    # -- lookups -------------------------------------------------------------------
    @staticmethod
    def _td_of(op):
        return op.forwarded.tensor.forwarded.tensor_description()

    def get_op_tensor(self, op):
        return self.op_tensors[self._td_of(op).base]

    def has_op_tensor(self, op):
        return self._td_of(op).base in self.op_tensors

    def get_op_tensor_view(self, op):
        return self.get_tensor_description_tensor_view(self._td_of(op))

    def get_tensor_view_value(self, op, host_tensor=None):
        return self.get_op_tensor_view(op).get(host_tensor)

    def get_tensor_description_tensor(self, tensor_description):
        return self.op_tensors[tensor_description.base]

    def has_tensor_description_tensor(self, tensor_description):
        return tensor_description.base in self.op_tensors

    def get_tensor_description_tensor_view(self, tensor_description):
        key = (tensor_description.base, tensor_description.parameter_key)
        view = self.op_tensor_views.get(key)
        if view is None:
            view = self.op_tensors[tensor_description.base].device_tensor(tensor_description)
            self.op_tensor_views[key] = view
            if self.allocated:
                view.transform_allocate()
        return view

    # -- host <-> device -------------------------------------------------------------
    def host_to_device(self, computation, parameters, args):
        for param, arg in zip(parameters, args):
            self.get_op_tensor_view(param)[...] = arg

    def device_to_host(self, computation, op, tensor=None):
        if self.has_op_tensor(op):
            return self.get_op_tensor_view(op).get(tensor)

    # -- hooks a backend provides -----------------------------------------------------
    def start_transform_allocate(self):
        raise NotImplementedError

    def finish_transform_allocate(self):
        raise NotImplementedError

    def transform_ordered_ops(self, computation, ordered_ops, name):
        raise NotImplementedError

    def finish_transform(self):
        raise NotImplementedError

    def allocate_storage(self):
        raise NotImplementedError

    def device_buffer_storage(self, bytes, dtype, name):
        raise NotImplementedError

    # -- flow ----------------------------------------------------------------------------
    def allocate(self):
        if self.allocated:
            return
        if not self.finalized:
            self._transform_computations()
        self.allocate_storage()
        self.allocated = True
        init_states = OrderedSet()
        for op in self.ops:
            op = op.forwarded
            for state in (op.states_read | op.states_written):
                state = state.forwarded
                if state.initial_value is not None:
                    init_states.add(state)
        for state in init_states:
            td = state.tensor.tensor_description()
            self.get_tensor_description_tensor_view(td)[...] = state.initial_value

    def add_computation(self, computation):
        if self.finalized:
            raise ValueError("Cannot create computations from a finalized transformer")
        computation = super(ComputationGraphTransformer, self).add_computation(computation)
        self.computations.add(computation)
        return computation

    def initialize(self):
        if self.initialized:
            return
        self.allocate()
        self.initialized = True

    def _transform_computations(self):
        all_results = [comp.computation_op for comp in self.computations]
        self.run_registered_graph_passes(ops=all_results)
        self.ops = Op.ordered_ops(all_results)

        def ensure_tensor(op):
            op = op.forwarded
            td = op.tensor_description()
            base = td.base
            if base not in self.op_tensors:
                tensor = self.device_buffer_storage(base.tensor_size, base.dtype, base.name)
                self.op_tensors[base] = tensor
                self.device_buffers.add(tensor)
            self.get_tensor_description_tensor_view(td)

        for op in self.ops:
            if op.is_tensor_op:
                ensure_tensor(op)
            # state tensors are reached through reads / writes, not through deps
            for state in (op.states_read | op.states_written):
                ensure_tensor(state)
        # a parameter nothing reads still receives its argument at every call
        for comp in self.computations:
            for param in comp.computation_op.parameters:
                ensure_tensor(param)

        self.start_transform_allocate()
        for device_buffer in self.device_buffers:
            device_buffer.transform_allocate()
        self.finish_transform_allocate()

        for comp in self.computations:
            comp.computation_name = self.transform_ordered_ops(
                comp, Op.ordered_ops([comp.computation_op]), name=comp.name)
        self.finish_transform()
        self.finalized = True


__transformer_factory = None


def make_transformer():
    """A transformer from the factory installed with set_transformer_factory (base.py:807-814)."""
    if __transformer_factory is None:
        raise ValueError("no transformer factory set; call set_transformer_factory first")
    return __transformer_factory()


def get_transformer_factory():
    """The factory make_transformer() currently uses (None when unset)."""
    return __transformer_factory


def set_transformer_factory(factory):
    global __transformer_factory
    __transformer_factory = factory


def transformer_choices():
    return sorted(Transformer.transformers.keys())


def allocate_transformer(name, **kargs):
    try:
        return Transformer.transformers[name](**kargs)
    except KeyError:
        names = ", ".join(["'%s'" % (_,) for _ in transformer_choices()])
        raise ValueError("transformer must be one of (%s)" % (names,))


def make_transformer_factory(name, **kargs):
    def factory():
        return allocate_transformer(name, **kargs)
    factory.name = name
    return factory
