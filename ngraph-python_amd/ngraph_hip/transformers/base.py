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

from ngraph_hip.op_graph.op_graph import Op, OrderedSet, computation as make_computation_op


class UnsupportedTransformerException(Exception):
    pass


class Computation(object):
    """What `transformer.computation(...)` returns: call it with the parameters' values
    (positionally, or `feed_dict={placeholder: value}`) and get the results back in the shape
    `returns` had (base.py:94-136)."""

    _serial = 0

    def __init__(self, transformer, computation_op, **kwargs):
        Computation._serial += 1
        self.name = "Computation_%d" % (Computation._serial - 1)
        self.transformer = transformer
        self.computation_op = computation_op
        self.computation_name = None        # set by the backend when it lowers the computation
        self.executor = None                # zero-argument callable, set by the backend

    def unpack_args_or_feed_dict(self, args, kwargs):
        """The parameter values in parameter order, from either calling convention."""
        wanted = self.computation_op.parameters
        if kwargs.get("feed_dict") is not None:
            feed = kwargs.pop("feed_dict")
            if args:
                raise ValueError("Can not supply both positional and feed_dict arguments "
                                 "to Computation")
            args = tuple(feed[p.tensor] for p in wanted)
        else:
            kwargs.pop("feed_dict", None)
        if len(args) != len(wanted):
            raise ValueError("Computation was expecting {expected} arguments, but was called "
                             "with {called}.".format(expected=len(wanted), called=len(args)))
        return args

    def _fetch(self, op):
        if not op.is_tensor_op or "skip_returns" in op.metadata:
            return None
        return self.transformer.device_to_host(self, op)

    def __call__(self, *args, **kwargs):
        values = self.unpack_args_or_feed_dict(args, kwargs)
        t, cop = self.transformer, self.computation_op
        t.initialize()
        t.host_to_device(self, cop.parameters, values)
        self.executor()
        kind = cop.returns_kind
        if kind == "op":
            return self._fetch(cop.returns)
        if kind == "sequence":
            return tuple(self._fetch(op) for op in cop.returns)
        if kind == "set":
            return {key: self._fetch(op) for key, op in cop.returns_map.items()}
        return None


class DeviceBufferStorage(object):
    """One allocation on the device; every view of it is a DeviceTensor made by the backend's
    `create_device_tensor` and kept per view description (base.py:140-210)."""

    def __init__(self, transformer, bytes, dtype, name=None, **kwargs):
        self.transformer = transformer
        self.name = name
        self.dtype = dtype
        self.bytes = bytes
        self._view_of = {}                  # TensorDescription.parameter_key -> DeviceTensor

    @property
    def views(self):
        return self._view_of.values()

    def device_tensor(self, tensor_description):
        key = tensor_description.parameter_key
        if key not in self._view_of:
            self._view_of[key] = self.create_device_tensor(tensor_description)
        return self._view_of[key]

    def transform_allocate_views(self):
        for view in list(self.views):
            view.transform_allocate()

    def transform_allocate(self):
        self.transform_allocate_views()

    def create_device_tensor(self, tensor_description):
        raise NotImplementedError


class DeviceTensor(object):
    """A view of a DeviceBufferStorage described by a TensorDescription (base.py:213-262).
    Backends implement allocation and the host-side reads and writes."""

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
    """A transformer class that carries a `transformer_name` is entered under that name in the
    registry shared by the whole hierarchy (base.py:265-279)."""

    def __init__(cls, name, bases, dict_):
        super(Transformer_ABC_Meta, cls).__init__(name, bases, dict_)
        registry = getattr(cls, "transformers", None)
        if registry is None:
            registry = cls.transformers = {}
        label = getattr(cls, "transformer_name", None)
        if label is not None:
            registry[label] = cls


class Transformer(object, metaclass=Transformer_ABC_Meta):
    """Turns op graphs into something that runs (base.py:282-475)."""

    default_rtol = 1e-05
    default_atol = 1e-08

    def __init__(self, **kwargs):
        super(Transformer, self).__init__()
        self.byte_alignment = 4
        self.graph_passes = []

    @classmethod
    def get_default_tolerance(cls, desired):
        return cls.default_atol, cls.default_rtol

    # -- computations ---------------------------------------------------------------------
    def make_computation(self, computation):
        return Computation(self, computation)

    def add_computation(self, computation):
        return self.make_computation(computation)

    def computation(self, results, *parameters):
        return self.add_computation(make_computation_op(results, *parameters))

    def initialize(self):
        pass

    # -- graph passes -----------------------------------------------------------------------
    def register_graph_pass(self, graph_pass, position=None):
        if position is None:
            position = len(self.graph_passes)
        self.graph_passes.insert(position, graph_pass)

    # -- diagnostics the reference offers and this backend does not produce -------------------
    def set_output_statistics_file(self, statistics_file):
        pass

    def save_output_statistics_file(self):
        pass

    def close(self):
        pass

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ComputationGraphTransformer(Transformer):
    """The flow every graph backend shares (base.py:478-801): collect computations; at the first
    use run the graph passes over all of them together, give every base tensor one device
    buffer and every tensor description a view, let the backend lower each computation
    (`transform_ordered_ops`), allocate, write initial values.  After that no computation can
    be added."""

    def __init__(self, **kwargs):
        super(ComputationGraphTransformer, self).__init__(**kwargs)
        self.computations = OrderedSet()
        self.ops = []
        self.finalized = self.allocated = self.initialized = False
        self.initialize_allocations()

    def initialize_allocations(self):
        self.device_buffers = OrderedSet()
        self.op_tensors = {}                 # base TensorDescription -> DeviceBufferStorage
        self.op_tensor_views = {}            # (base, view key) -> DeviceTensor

    def run_registered_graph_passes(self, ops, **kwargs):
        for one_pass in self.graph_passes:
            one_pass.wrapped_do_pass(ops=ops, **kwargs)
        return ops

    # -- hooks a backend provides -----------------------------------------------------------
    def device_buffer_storage(self, bytes, dtype, name):
        raise NotImplementedError

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

    # -- from ops and tensor descriptions to storage and views ----------------------------------
    @staticmethod
    def _td_of(op):
        return op.forwarded.tensor.forwarded.tensor_description()

    def has_tensor_description_tensor(self, tensor_description):
        return tensor_description.base in self.op_tensors

    def get_tensor_description_tensor(self, tensor_description):
        return self.op_tensors[tensor_description.base]

    def get_tensor_description_tensor_view(self, tensor_description):
        key = (tensor_description.base, tensor_description.parameter_key)
        if key not in self.op_tensor_views:
            view = self.get_tensor_description_tensor(tensor_description).device_tensor(tensor_description)
            self.op_tensor_views[key] = view
            if self.allocated:               # a view asked for after allocation: bring it up now
                view.transform_allocate()
        return self.op_tensor_views[key]

    def has_op_tensor(self, op):
        return self.has_tensor_description_tensor(self._td_of(op))

    def get_op_tensor(self, op):
        return self.get_tensor_description_tensor(self._td_of(op))

    def get_op_tensor_view(self, op):
        return self.get_tensor_description_tensor_view(self._td_of(op))

    def get_tensor_view_value(self, op, host_tensor=None):
        return self.get_op_tensor_view(op).get(host_tensor)

    # -- host <-> device ------------------------------------------------------------------------
    def host_to_device(self, computation, parameters, args):
        for parameter, value in zip(parameters, args):
            self.get_op_tensor_view(parameter)[...] = value

    def device_to_host(self, computation, op, tensor=None):
        return self.get_op_tensor_view(op).get(tensor) if self.has_op_tensor(op) else None

    # -- flow -------------------------------------------------------------------------------------
    def add_computation(self, computation):
        if self.finalized:
            raise ValueError("Cannot create computations from a finalized transformer")
        handle = super(ComputationGraphTransformer, self).add_computation(computation)
        self.computations.add(handle)
        return handle

    def initialize(self):
        if not self.initialized:
            self.allocate()
            self.initialized = True

    def allocate(self):
        if self.allocated:
            return
        if not self.finalized:
            self._transform_computations()
        self.allocate_storage()
        self.allocated = True
        self._write_initial_values()

    @staticmethod
    def _states_of(op):
        """The state tensors an op reads or writes (reached through these sets, not through
        the op's dependencies)."""
        for state in (op.states_read | op.states_written):
            yield state.forwarded

    def _write_initial_values(self):
        with_value = OrderedSet()
        for op in self.ops:
            for state in self._states_of(op.forwarded):
                if state.initial_value is not None:
                    with_value.add(state)
        for state in with_value:
            view = self.get_tensor_description_tensor_view(state.tensor.tensor_description())
            view[...] = state.initial_value

    def _claim_storage(self, op):
        """A device buffer for the op's base tensor (once) and a view for its description."""
        description = op.forwarded.tensor_description()
        base = description.base
        if base not in self.op_tensors:
            storage = self.device_buffer_storage(base.tensor_size, base.dtype, base.name)
            self.op_tensors[base] = storage
            self.device_buffers.add(storage)
        self.get_tensor_description_tensor_view(description)

    def _transform_computations(self):
        roots = [handle.computation_op for handle in self.computations]
        self.run_registered_graph_passes(ops=roots)
        self.ops = Op.ordered_ops(roots)
        for op in self.ops:
            if op.is_tensor_op:
                self._claim_storage(op)
            for state in (op.states_read | op.states_written):
                self._claim_storage(state)
        # a parameter nothing reads still receives its argument at every call
        for root in roots:
            for parameter in root.parameters:
                self._claim_storage(parameter)

        self.start_transform_allocate()
        for storage in self.device_buffers:
            storage.transform_allocate()
        self.finish_transform_allocate()

        for handle in self.computations:
            ops_of_handle = Op.ordered_ops([handle.computation_op])
            handle.computation_name = self.transform_ordered_ops(handle, ops_of_handle, name=handle.name)
        self.finish_transform()
        self.finalized = True


# ---------------------------------------------------------------------------------- factories
_factory = None


def set_transformer_factory(factory):
    """Install the factory make_transformer() uses (base.py:817-825)."""
    global _factory
    _factory = factory


def get_transformer_factory():
    """The factory make_transformer() currently uses (None when unset)."""
    return _factory


def make_transformer():
    """A transformer from the factory installed with set_transformer_factory (base.py:807-814)."""
    if _factory is None:
        raise ValueError("no transformer factory set; call set_transformer_factory first")
    return _factory()


def transformer_choices():
    return sorted(Transformer.transformers)


def allocate_transformer(name, **kargs):
    """An instance of the transformer registered as `name` (base.py:834-840)."""
    cls = Transformer.transformers.get(name)
    if cls is None:
        raise ValueError("transformer must be one of (%s)" %
                         ", ".join("'%s'" % choice for choice in transformer_choices()))
    return cls(**kargs)


def make_transformer_factory(name, **kargs):
    """A zero-argument factory for transformer `name`, tagged with `.name` (base.py:843-847)."""
    def factory():
        return allocate_transformer(name, **kargs)
    factory.name = name
    return factory
