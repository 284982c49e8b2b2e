"""`flexhip`: the flex16 variant of the HIP transformer.

Mirrors ngraph/transformers/flexgputransform.py:

* every tensor op gets the flex dtype (FlexDtypePass, passes/flexpass.py:24-29), every
  device buffer a flex entry (flexgputransform.py:211-217);
* before each kernel the entries' scales are bound into the kernel arguments and the
  output statistics words cleared, after each kernel max|mantissa| comes back and the
  manager updates the exponent (flexgputransform.py:56-61, 347-366);
* host writes quantise on the host (divide by scale, clip, truncate), host reads
  dequantise (flexgputransform.py:178-208);
* tolerances: rtol 1e-2, atol 8 x scale(max|desired|) (flexgputransform.py:80-103).

What differs from the reference by design: elementwise chains run as ONE fused
kernel, so intermediates stay fp32 registers and only the group's outputs are
rounded to flex16 (the reference launches one kernel, and one rounding, per op);
`fusion=False` restores the per-op behaviour the reference's known-answer vectors
were recorded with.  A fresh output tensor's first exponent comes from a probe
launch that measures the result's true range without storing anything.
"""
from __future__ import division

import numpy as np

from ngraph_hip.flex import HipFlexManager, hipflex16, HipFlex
from ngraph_hip.flex.base import flex_gpu_transformer_name
from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.runtime.hiplib import NGH_FLEX16, NGH_SPEC_PROBE, OPCODES
from ngraph_hip.transformers.hiptransform import (HipTransformer, HipDeviceTensor,
                                                  HipDeviceBufferStorage, HipKernelGroup,
                                                  FusedKernel, CopyKernel, ChainKernel, _td)
from ngraph_hip.transformers.passes.passes import PeepholeGraphPass


class FlexDtypePass(PeepholeGraphPass):
    """Every tensor op computes in flex16 (passes/flexpass.py:24-29)."""

    def do_pass(self, ops, **kwargs):
        for op in og.Op.ordered_ops(ops):
            op = op.forwarded
            states = list(op.states_read) + list(op.states_written)
            for t in [op] + states:
                if t.is_tensor_op and not isinstance(t, og.ValueOp):
                    if not isinstance(t.dtype, HipFlex):
                        t.dtype = hipflex16
                        if hasattr(t, "invalidate_tensor_description"):
                            t.invalidate_tensor_description()


class FlexHipDeviceTensor(HipDeviceTensor):
    """Flex scale-aware device tensor (flexgputransform.py:160-208)."""

    @property
    def scale(self):
        return self.flex_entry.scale

    @property
    def flex_entry(self):
        return self.device_buffer.flex_entry

    def get(self, tensor):
        raw = self._read_raw()
        value = (raw.astype(np.float32) * np.float32(self.scale)).astype(np.float32)
        if tensor is None:
            return value
        tensor[...] = value
        return tensor

    def __setitem__(self, key, value):
        if not (key is Ellipsis or key == () or key == slice(None, None, None)):
            whole = self.get(None)
            whole[key] = value
            value = whole
        value = np.asarray(value, dtype=np.float64)
        entry = self.flex_entry
        # though not a kernel, a host write modifies tensor values: manage the exponent
        entry.manage_before_computation(value)
        scaled = value / entry.scale
        bits = entry.dtype.storage_bits - 1
        scaled = np.clip(scaled, -2 ** bits, 2 ** bits - 1)
        mantissa = scaled.astype(np.int16)                 # truncation, as astype does
        self._write_raw(mantissa)
        maxabs = int(np.amax(np.absolute(mantissa.astype(np.int32)))) if mantissa.size else 0
        entry.manage_after_computation(maxabs, self.transformer.flex_manager.autoflex_count)


class FlexHipDeviceBufferStorage(HipDeviceBufferStorage):
    def __init__(self, transformer, bytes, dtype, **kwargs):
        super(FlexHipDeviceBufferStorage, self).__init__(transformer, bytes, dtype, **kwargs)
        self.flex_entry = transformer.flex_manager.make_flex_entry(name=self.name)

    def create_device_tensor(self, tensor_description):
        return FlexHipDeviceTensor(self.transformer, self, tensor_description,
                                   name="v_" + tensor_description.name)


class FlexManaged(object):
    """What the kernel group's flex management needs of a kernel that has `specs`,
    `flex_bindings` [(spec index, operand slot, flex entry, is written)],
    `output_flex_entries` and `in_place_flex_ids`."""

    @property
    def output_flex_ids(self):
        return [e.flex_id for e in self.output_flex_entries]

    def bind_flex_scales(self):
        """Host-managed mode: the current scales travel as kernel arguments, rebound before
        every launch (flexgputransform.py:56-61)."""
        for index, slot, entry, is_output in self.flex_bindings:
            t = self.specs[index].tensors[slot]
            t.scale = entry.scale
            t.dev_scale = None
            t.dev_stats = entry.ptr if is_output else None

    def bind_flex_state_pointers(self):
        """Device-resident mode: kernels read scales from the state table; bound once."""
        if getattr(self, "_state_bound", False):
            return
        for index, slot, entry, is_output in self.flex_bindings:
            t = self.specs[index].tensors[slot]
            t.dev_scale = entry.scale_ptr
            t.dev_stats = entry.ptr if is_output else None
        self._state_bound = True

    def execute_managed(self, rt, dev_table, count):
        self.bind_flex_state_pointers()
        if not hasattr(self, "_id_arrays"):
            ids = [e.flex_id for e in self.output_flex_entries]
            in_place = [1 if i in self.in_place_flex_ids else 0 for i in ids]
            self._id_lists = (ids, in_place)
            self._id_arrays = rt.make_id_arrays(ids, in_place)
        if len(self.specs) == 1:
            rt.launch_fused_flex(self.specs[0], dev_table, self._id_arrays, count)
            return
        # several launches cover one set of tensors (an outer axis looped on the host): one
        # exponent for all of them, statistics merged over all of them
        ids, in_place = self._id_lists
        rt.flex_prepare(dev_table, ids, in_place)
        for spec in self.specs:
            rt.launch_fused(spec)
        rt.flex_update(dev_table, ids, count)


class FlexFusedKernel(FlexManaged, FusedKernel):
    """Fused kernel whose operands carry flex scales and statistics words."""

    def __init__(self, *args, **kwargs):
        super(FlexFusedKernel, self).__init__(*args, **kwargs)
        self.output_flex_entries = []

    fill_store = "store_trunc"   # FlexFillKernel: int(value / scale), clipped (tensor_ops.py:690-707)

    def _constant_value(self, value):
        """A scalar constant as the host write path would have stored it: tightest-fit
        exponent, truncated mantissa (flexgputransform.py:183-203)."""
        dec = hipflex16.fit_dec(value)
        if dec is None:
            return 0.0
        scale = 1.0 / 2 ** dec
        m = int(np.clip(np.float64(value) / scale, hipflex16.nclip, hipflex16.pclip))
        return float(m * scale)

    def bind_buffers(self):
        super(FlexFusedKernel, self).bind_buffers()
        seen, entries, read_ids = set(), [], set()
        for index, slot, entry, is_output in self.flex_bindings:
            if is_output and entry.flex_id not in seen:
                seen.add(entry.flex_id)
                entries.append(entry)
            spec = self.specs[index]
            if any(o.opcode == 1 and o.a == slot for o in spec.ops[:spec.n_ops]):
                read_ids.add(entry.flex_id)
        self.output_flex_entries = entries
        self.in_place_flex_ids = set(e.flex_id for e in entries) & read_ids

    def probe(self):
        """Measure max|fp32 result| of every not yet initialised output without storing."""
        fresh = [e for e in self.output_flex_entries if not e.initialized]
        if not fresh:
            return
        rt = self.transformer.runtime
        for e in self.output_flex_entries:
            rt.stats_reset(e.ptr, 1)
        self.bind_flex_scales()
        for spec in self.specs:
            spec.flags |= NGH_SPEC_PROBE
            try:
                rt.launch_fused(spec)
            finally:
                spec.flags &= ~NGH_SPEC_PROBE
        for e in fresh:
            bits = rt.stats_read(e.ptr, 1)
            e.init_from_value(float(bits.view(np.float32)[0]))


class FlexCopyKernel(CopyKernel):
    """A copy moves mantissas verbatim, so the copy shares its source's flex entry
    (FlexPropagateEntryPass, passes/flexpass.py:32-50)."""

    output_flex_entries = ()

    def bind_flex_state_pointers(self):
        pass

    def execute_managed(self, rt, dev_table, count):
        self.execute()

    def bind_buffers(self):
        t = self.transformer
        src_buf = t.op_tensors[_td(self.op.args[0].forwarded).base]
        dst_buf = t.op_tensors[_td(self.op).base]
        dst_buf.flex_entry = src_buf.flex_entry
        super(FlexCopyKernel, self).bind_buffers()

    def probe(self):
        pass


class FlexChainKernel(FlexManaged, ChainKernel):
    """Consecutive flex kernels over the same rows as the stages of one spec, one launch when the
    library has the chain's program: a softmax's maximum, sum of exponentials and result, each a
    flex16 tensor with an exponent of its own.  One prepare / launch / update covers all of them.
    A stage reads what an earlier stage wrote from memory, rounded as stored, so the chain leaves
    the bits its members leave when they run one by one -- which they do until every output has
    its first exponent (a member's probe needs its predecessors' results) and while the library
    has no program for the chain."""

    def __init__(self, transformer, members, spec, uses, operands=()):
        super(FlexChainKernel, self).__init__(transformer, members, spec, uses, operands)
        t = transformer
        self.flex_bindings = []
        for s, td in enumerate(self.operands):
            entry = t.flex_entry_of(td)
            if entry is not None:
                self.flex_bindings.append((0, s, entry, uses[s][2]))
        # an output holds data from before the launch that the chain reads when a stage loads it
        # no later than the first stage that writes it
        load, store = OPCODES["load"], OPCODES["store"]
        first_load, first_write = {}, {}
        for stage in range(spec.n_stages):
            st = spec.stages[stage]
            for o in spec.ops[st.op_begin:st.op_end]:
                if o.opcode == load:
                    first_load.setdefault(o.a, stage)
                elif o.opcode == store:
                    first_write.setdefault(o.dst, stage)
            for r in range(st.n_reductions):
                first_write.setdefault(st.red_out[r], stage)
        seen, entries, in_place = set(), [], set()
        for _, slot, entry, is_output in self.flex_bindings:
            if not is_output:
                continue
            if entry.flex_id not in seen:
                seen.add(entry.flex_id)
                entries.append(entry)
            if slot in first_load and first_load[slot] <= first_write.get(slot, spec.n_stages):
                in_place.add(entry.flex_id)
        self.output_flex_entries = entries
        self.in_place_flex_ids = in_place

    def active(self):
        """One launch, managed as one kernel?  Else the members run, each managed by itself.
        (Asked before every execution: once true it stays true, and looking at a record reads
        the state table back from the device.)"""
        if not getattr(self, "_active", False):
            self._active = self.ready and all(e.initialized for e in self.output_flex_entries)
        return self._active

    @property
    def _all_initialized(self):
        return True            # (only asked of an active chain)

    @_all_initialized.setter
    def _all_initialized(self, value):
        pass

    def probe(self):
        pass


class FlexHipKernelGroup(HipKernelGroup):
    """Flex management around every kernel (flexgputransform.py:224-371)."""

    def setup_kernel_execute(self, kernel):
        manager = self.transformer.flex_manager
        if manager.resident and not getattr(kernel, "_all_initialized", False):
            kernel.probe()
            kernel._all_initialized = all(e.initialized for e in kernel.output_flex_entries)
        elif not manager.resident:
            kernel.probe()
        manager.manage_before_computation(kernel)
        if manager.resident:
            kernel.bind_flex_state_pointers()
        else:
            kernel.bind_flex_scales()

    def after_kernel_execute(self, kernel):
        self.transformer.flex_manager.manage_after_computation(kernel)

    def __call__(self):
        manager = self.transformer.flex_manager
        manager.autoflex_count += 1
        if self._programs is not None and self._programs.poll():
            # (kernels compiled in the background are loaded by the thread that owns the runtime)
            self._programs = None
            self.programs_changed()
        if manager.resident and getattr(self, "_steady", False):
            # steady state of the device-resident mode: every tensor initialised, pointers
            # bound; one library call per kernel does prepare + launch + policy update
            manager.push()
            rt, count = self.transformer.runtime, manager.autoflex_count
            for k in self.execution_units():
                k.execute_managed(rt, manager.dev_table, count)
            manager.device_dirty = True
            return
        super(FlexHipKernelGroup, self).__call__()
        if manager.resident:
            units = list(self.execution_units())
            self._steady = all(getattr(k, "_all_initialized", False) or not k.output_flex_entries
                               for k in units) and \
                all(isinstance(k, (FlexFusedKernel, FlexCopyKernel, FlexChainKernel)) for k in units)

    def execution_units(self):
        """A chain that is not one launch yet stands for its members."""
        for k in self.kernels:
            if isinstance(k, FlexChainKernel) and not k.active():
                for m in k.members:
                    yield m
            else:
                yield k

    @property
    def output_flex_ids(self):
        ids = []
        for k in self.kernels:
            ids.extend(getattr(k, "output_flex_ids", []))
        return ids


class FlexHipTransformer(HipTransformer):
    """Flex specifics: a flex manager, flex-aware buffers / tensors / kernel group."""

    transformer_name = flex_gpu_transformer_name
    fixed_point_res = HipFlexManager.fixed_point_resolution()
    default_rtol = 1e-02
    atol_precision_multiplier = 8
    kernel_group_class = FlexHipKernelGroup
    chain_member_class = FlexFusedKernel
    chain_kernel_class = FlexChainKernel
    max_written_views = 4        # a kernel merges max|mantissa| for at most 4 flex results
    split_reductions = False     # an intermediate result would be rounded to flex16 on its way

    def __init__(self, fixed_point=False, flex_verbose=False, collect_flex_data=False,
                 resident=True, **kwargs):
        """resident=True (the default) keeps scales, statistics and the exponent policy on the
        device: no host round trip per kernel, a record is read back only when the host looks at
        its tensor.  resident=False follows the reference's loop, which reads max|mantissa| back
        and runs the policy on the host after every kernel (flexgputransform.py:347-366); both
        modes leave the same state after every computation."""
        self.flex_manager = HipFlexManager(fixed_point=fixed_point, verbose=flex_verbose,
                                           resident=resident)
        kwargs.setdefault("fuse_moments", False)
        super(FlexHipTransformer, self).__init__(**kwargs)
        self.flex_manager.runtime = self.runtime
        self.fixed_point = fixed_point
        self.collect_flex_data = collect_flex_data
        self.register_graph_pass(FlexDtypePass())

    @classmethod
    def get_default_tolerance(cls, desired):
        desired = np.asarray(desired, dtype=np.float64)
        scale = hipflex16.get_scale(np.max(np.abs(desired)) if desired.size else 0.0)
        return scale * cls.atol_precision_multiplier, cls.default_rtol

    def set_output_statistics_file(self, statistics_file):
        if self.collect_flex_data:
            self.flex_manager.set_h5py_file(statistics_file)

    def save_output_statistics_file(self):
        if self.collect_flex_data:
            self.flex_manager.save_diagnostic_data()

    def ngh_dtype(self, dtype):
        if isinstance(dtype, HipFlex):
            return NGH_FLEX16
        return super(FlexHipTransformer, self).ngh_dtype(dtype)

    def storage_dtype(self, dtype):
        if isinstance(dtype, HipFlex):
            return dtype.storage_dtype
        raise NotImplementedError

    def flex_entry_of(self, tensor_description):
        buf = self.op_tensors.get(tensor_description.base)
        return getattr(buf, "flex_entry", None)

    def device_buffer_storage(self, bytes, dtype, name):
        return FlexHipDeviceBufferStorage(self, bytes, dtype, name="a_" + name)

    def make_fused_kernel(self, ops, store_ops, name):
        return FlexFusedKernel(self, ops, store_ops, name)

    def make_copy_kernel(self, op):
        return FlexCopyKernel(self, op)

    def transform_ordered_ops(self, computation, ordered_ops, name):
        ret = super(FlexHipTransformer, self).transform_ordered_ops(computation, ordered_ops, name)
        self.flex_manager.allocate(self.runtime)
        return ret
