"""`hipgpu`: the MI355X transformer for fused elementwise / reduction graphs.

Plays the part of ngraph/transformers/gputransform.py for this path:

* `kernel_op_name` maps each op class to a kernel op name the way
  `ElementWiseKernel.add_op` does (gputransform.py:124-275);
* `FusionPlanner` groups consecutive elementwise ops (optionally ended by
  reductions) that share an iteration space into one kernel spec.  The
  reference generator supports such compounds (float_ew2.py:553-612,
  1135-1429) but its transformer hands it one op at a time
  (gputransform.py:381-391); `fusion=False` reproduces that;
* operands become (pointer, element strides) views over at most three merged
  axes (float_ew2.py:289-338, MAX_AXES = 3), reductions see the reduced axes
  first (gputransform.py:117-122);
* `HipKernelGroup.__call__` is the executor loop (gputransform.py:508-522);
* `HipDeviceBufferStorage` / `HipDeviceTensor` own device memory and do host
  I/O, strided views going through the device copy kernel
  (gputransform.py:525-909).

The parts live in modules of their own: `hipdevice` (device memory, host I/O), `hiplowering`
(op names, operands, programs, `FusedKernel`), `hipmoments` (one-pass statistics), `hipchains`
(several kernels as the stages of one launch), `hipplanner` (which ops share a kernel); this
module holds the executor loop and the transformer, and re-exports the names others import.

All arithmetic runs in libngraph_hip.so; if the library or a GPU is missing,
constructing the transformer raises.
"""
from __future__ import division

import os
from collections import OrderedDict

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.runtime.hiplib import (HipRuntime, DryRunRuntime, HipLibraryError, NGH_F32,
                                       NGH_FLEX16, NGH_I32, NGH_F16, NGH_U32, NGH_I16, NGH_I8, NGH_U8,
                                       NGH_MAX_TENSORS, NGH_CACHE_STREAM_LOAD, NGH_CACHE_STREAM_STORE)
from ngraph_hip.transformers.base import ComputationGraphTransformer, UnsupportedTransformerException
from ngraph_hip.transformers.passes.passes import SimplePrune
from ngraph_hip.transformers.passes.hippasses import TensorSizeFold, ReductionLayoutPass, ConstantFoldPass
from ngraph_hip.transformers.hipdevice import HipDeviceBufferStorage, HipDeviceTensor, _td, _adapt_td  # noqa: F401
from ngraph_hip.transformers.hiplowering import (FusedKernel, CopyKernel, HipKernel, kernel_op_name,  # noqa: F401
                                                 is_fusable, iteration_axes, og_unsupported)
from ngraph_hip.transformers.hipmoments import MomentsOp, MomentsFusionPass, MomentsKernel, moments_layout  # noqa: F401
from ngraph_hip.transformers.hipchains import ChainKernel, KernelRun  # noqa: F401
from ngraph_hip.transformers.hipplanner import FusionPlanner


class HipKernelGroup(object):
    """The kernels of one computation and the loop that runs them (gputransform.py:348-522)."""

    def __init__(self, transformer, name):
        self.transformer = transformer
        self.name = name
        self.kernels = []
        self._bound = False

    def bind(self):
        """Lower every kernel, then tell each operand what the rest of the computation does
        with its buffer (the cache hints of the C ABI)."""
        if self._bound:
            return
        for k in self.kernels:
            if not k.buffers_bound:
                k.bind_buffers()
        # (a run of kernels has settled which of them merge: its kernels take its place)
        self.kernels = [u for k in self.kernels for u in (k.kernels if isinstance(k, KernelRun) else [k])]
        self.assign_cache_hints()
        mode = self.transformer.jit
        if mode is True:
            # compile what would otherwise run on the interpreter (float_ew2.py:1553-1653: the
            # reference compiles every kernel of a computation at this point)
            from ngraph_hip.runtime import jit
            jit.ensure_programs(self.transformer.runtime, self.kernels, self.name,
                                min_elements=self.transformer.jit_min_elements)
            self.programs_changed()
        elif mode == "auto":
            # the same for the stages over large tensors, off the launch path: the computation
            # starts on the interpreter and picks the compiled kernels up when they are ready
            from ngraph_hip.runtime import jit
            self._programs = jit.start_background(self.transformer.runtime, self.kernels, self.name,
                                                  min_elements=self.transformer.jit_auto_min_elements,
                                                  small_min_elements=self.transformer.jit_min_elements,
                                                  after_calls=self.transformer.jit_after_calls)
        self._bound = True

    _programs = None

    def programs_changed(self):
        for k in self.kernels:
            if hasattr(k, "programs_changed"):
                k.programs_changed()
        self.drop_graph()            # (recorded launches name the kernels of before)
        self._pairs = None

    # -- the launches as one HIP graph (off unless the transformer is given graphs=True) -------
    # A computation of a few small kernels spends its time on launches.  With graphs=True its
    # launches are recorded once, after `graph_after_calls` ordinary executions (ngh_graph_begin /
    # _end), and replayed with one call from then on; two consecutive kernels that touch no common
    # buffer one of them writes are recorded side by side, so the device may run them together (an
    # LSTM cell and the column sum for its bias gradient).  Only kernels whose arguments are the
    # same in every execution are recorded (no random fills, no flex exponents), and only small
    # ones.  Off by default because it measured slower here: the LSTM step of two 4 us kernels
    # takes 10.6 us as two launches, 18.3 us as a graph of two nodes in a row and 31.4 us with the
    # nodes side by side.
    graph_after_calls = 2
    graph_max_elements = 1 << 21            # per kernel
    _graph = None
    _graph_calls = 0
    _graph_refused = False

    def drop_graph(self):
        graph, self._graph = self._graph, None
        self._graph_calls = 0
        if graph is not None and self.transformer.runtime is not None:
            self.transformer.runtime.graph_free(graph)

    def _graph_eligible(self):
        t = self.transformer
        if self._graph_refused or self._programs is not None:
            return False             # (while kernels are being compiled the launches may still change)
        if not t.graphs or type(self) is not HipKernelGroup or not getattr(t.runtime, "graphs", False) or \
                len(self.kernels) < 2:
            self._graph_refused = True
            return False
        for k in self.kernels:
            recordable = type(k) in (FusedKernel, ChainKernel) and not getattr(k, "n_rng_streams", 0) and \
                not any(getattr(m, "n_rng_streams", 0) for m in getattr(k, "members", ())) and \
                all(spec.shape[0] * spec.shape[1] * spec.shape[2] <= self.graph_max_elements for spec in k.specs)
            if not recordable:
                self._graph_refused = True
                return False
        return True

    @staticmethod
    def _independent(a, b):
        """Neither kernel writes a buffer the other touches."""
        def sets(k):
            uses = k.buffer_uses()
            return set(base for base, _, w in uses if w), set(base for base, _, _ in uses)
        wa, ua = sets(a)
        wb, ub = sets(b)
        return not (wa & ub) and not (wb & ua)

    def _record_graph(self):
        rt = self.transformer.runtime
        rt.graph_begin()
        try:
            ks, i = self.kernels, 0
            while i < len(ks):
                if i + 1 < len(ks) and self._independent(ks[i], ks[i + 1]):
                    rt.graph_fork()
                    ks[i].execute()
                    rt.graph_side(True)
                    ks[i + 1].execute()
                    rt.graph_join()
                    i += 2
                else:
                    ks[i].execute()
                    i += 1
            self._graph = rt.graph_end()
        except Exception:
            rt.graph_abandon()
            self._graph_refused = True          # (this computation stays with ordinary launches)

    def wait_for_programs(self, timeout=None):
        """Block until the kernels being compiled for this computation (jit="auto") are loaded;
        returns the compiler's message if it failed, else None."""
        if not self._bound:
            self.bind()
        if self._programs is None:
            return None
        self._programs.wait(timeout)
        error = self._programs.error
        self._programs = None
        self.programs_changed()
        return error

    def cancel_programs(self):
        if self._programs is not None:
            self._programs.cancel()
            self._programs = None

    def assign_cache_hints(self):
        uses = [k.buffer_uses() for k in self.kernels]
        readers = {}
        for i, ku in enumerate(uses):
            for base, is_read, _ in ku:
                if is_read:
                    readers.setdefault(base, set()).add(i)
        for i, k in enumerate(self.kernels):
            def hint_of(base, is_read, is_written, i=i):
                hint = 0
                r = readers.get(base, set())
                if is_read and r == {i}:
                    hint |= NGH_CACHE_STREAM_LOAD
                # a result that nothing here reads again; state updated in place is read by
                # the next execution and stays cacheable
                if is_written and not is_read and not any(j > i for j in r) \
                        and not getattr(base, "is_persistent", False):
                    hint |= NGH_CACHE_STREAM_STORE
                return hint
            k.set_cache_hints(hint_of)

    def setup_kernel_execute(self, kernel):
        pass

    def after_kernel_execute(self, kernel):
        pass

    def __call__(self):
        if not self._bound:
            self.bind()
        if self._programs is not None and self._programs.poll():
            self._programs = None
            self.programs_changed()
        if self._graph is not None:
            self.transformer.runtime.graph_launch(self._graph)
            return
        if self._pairs is None:
            self._pairs = self._find_pairs()
        if self._pairs:
            self._execute_with_pairs()
        else:
            for k in self.execution_units():
                self.setup_kernel_execute(k)
                k.execute()
                self.after_kernel_execute(k)
        self._graph_calls += 1
        if self._graph_calls >= self.graph_after_calls and not self._graph_refused and self._graph_eligible():
            self._record_graph()

    def execution_units(self):
        """The kernels in the order they are launched."""
        return self.kernels

    # -- two independent kernels in one launch -------------------------------------------------
    # Consecutive fused kernels that touch no common buffer one of them writes go to the library
    # in one call (ngh_launch_fused_pair), which runs them as ONE launch when it has their programs
    # built as a pair (an LSTM cell and the column sum for its bias gradient).  A pair the library
    # launches one by one anyway is not tried again.
    _pairs = None                # {index of the first kernel of a pair}

    def _find_pairs(self):
        pairs = set()
        if type(self) is not HipKernelGroup or not hasattr(self.transformer.runtime, "launch_fused_pair"):
            return pairs
        ks, i = self.kernels, 0
        plain = lambda k: type(k) is FusedKernel and len(k.specs) == 1 and not k.n_rng_streams
        while i + 1 < len(ks):
            if plain(ks[i]) and plain(ks[i + 1]) and self._independent(ks[i], ks[i + 1]):
                pairs.add(i)
                i += 2
            else:
                i += 1
        return pairs

    def _execute_with_pairs(self):
        rt, ks, i = self.transformer.runtime, self.kernels, 0
        while i < len(ks):
            if i in self._pairs:
                if not rt.launch_fused_pair(ks[i].specs[0], ks[i + 1].specs[0]):
                    self._pairs.discard(i)
                i += 2
            else:
                ks[i].execute()
                i += 1

    def profile(self, repeats=1, inner=1):
        """Per-kernel durations from HIP events on the launch stream.

        Each kernel is launched `inner` times back to back between one pair of events and the
        elapsed time divided by `inner` (amortises the event and launch overhead, so the
        figure is comparable with a profiler's kernel duration); this is repeated `repeats`
        times.  Returns [(kernel, [ms per launch])].  Kernels run out of their normal
        interleaving, so use it for per-kernel time, not for end-to-end time."""
        rt = self.transformer.runtime
        if not self._bound:
            self.bind()
        units = list(self.execution_units())
        times = [[] for _ in units]
        for _ in range(repeats):
            for i, k in enumerate(units):
                self.setup_kernel_execute(k)
                rt.timer_begin()
                for _ in range(inner):
                    k.execute()
                times[i].append(rt.timer_end() / inner)
                self.after_kernel_execute(k)
        return list(zip(units, times))


class HipTransformer(ComputationGraphTransformer):
    """Transformer for executing graphs on an MI355X through libngraph_hip.so."""

    transformer_name = "hipgpu"
    default_rtol = 1e-05
    default_atol = 1e-08

    kernel_group_class = HipKernelGroup
    max_written_views = NGH_MAX_TENSORS      # results one fused kernel may write
    split_reductions = True                  # ReductionLayoutPass: reduce group by group of axes, no copy
    chain_kernels = True                     # consecutive kernels over the same rows run as stages of one spec
    chain_member_class = FusedKernel         # (the kernels that may merge, and what they merge into)
    chain_kernel_class = ChainKernel

    def __init__(self, device_id=0, fusion=True, dry_run=False, fuse_moments=None, rng_seed=0, jit=None,
                 jit_min_elements=4096, jit_auto_min_elements=1 << 22, jit_after_calls=0, graphs=None, **kwargs):
        """dry_run=True lowers graphs to kernel specs without a device (no results can be
        read back); it exists so the host-side lowering can be inspected and tested.
        rng_seed keys the random fills (ng.uniform / ng.normal): same seed, same numbers.
        jit: how stages that the library has no compiled program for get one (the reference
        compiles every kernel of a computation when it is initialised, float_ew2.py:1553-1653).
        "auto" (the default unless NGH_JIT says otherwise): stages of at least
        jit_auto_min_elements elements are compiled in the background and swapped in when
        ready; True: every stage of at least jit_min_elements elements is compiled before the
        first launch; False: never.
        graphs: record the launches of computations of a few small kernels as one HIP graph
        after their first executions (default: off unless NGH_GRAPHS=1; replaying a graph of two
        small kernels measured slower than launching them)."""
        self.graphs = (os.environ.get("NGH_GRAPHS", "0") == "1") if graphs is None else bool(graphs)
        from ngraph_hip.runtime import jit as _jit
        self.jit = _jit.normalize_mode(jit)
        self.jit_min_elements = int(jit_min_elements)
        self.jit_auto_min_elements = int(jit_auto_min_elements)
        self.jit_after_calls = int(jit_after_calls)
        try:
            self.runtime = DryRunRuntime() if dry_run else HipRuntime(device_id)
        except HipLibraryError as e:
            raise UnsupportedTransformerException("hipgpu needs libngraph_hip.so and an MI355X: %s" % e)
        super(HipTransformer, self).__init__(**kwargs)
        self.fusion = fusion
        self.rng_seed = int(rng_seed)
        self.n_kernels = 0
        self.kernel_groups = OrderedDict()
        self.graph_passes = [SimplePrune(), TensorSizeFold(), ConstantFoldPass(), SimplePrune()]
        if fusion if fuse_moments is None else fuse_moments:
            self.graph_passes.append(MomentsFusionPass())
        self.graph_passes.append(ReductionLayoutPass(split=self.split_reductions))

    # -- dtype mapping ---------------------------------------------------------------------
    def ngh_dtype(self, dtype):
        if not isinstance(dtype, np.dtype):
            return NGH_FLEX16
        # float_ew2.py:615-641 lists the storage types a compound kernel may touch
        for np_type, code in ((np.float32, NGH_F32), (np.int32, NGH_I32), (np.float16, NGH_F16),
                              (np.uint32, NGH_U32), (np.int16, NGH_I16), (np.int8, NGH_I8),
                              (np.uint8, NGH_U8)):
            if dtype == np_type:
                return code
        raise TypeError("hipgpu: unsupported tensor dtype %s" % dtype)

    def flex_entry_of(self, tensor_description):
        return None

    # -- hooks ---------------------------------------------------------------------------------
    def device_buffer_storage(self, bytes, dtype, name):
        return HipDeviceBufferStorage(self, bytes, dtype, name="a_" + name)

    def start_transform_allocate(self):
        pass

    def finish_transform_allocate(self):
        pass

    def gpu_kernel_group(self, name):
        return self.kernel_group_class(self, name)

    def _usage_maps(self):
        """Which device ops read each buffer, over every computation of this transformer."""
        readers, returned = {}, set()
        for op in self.ops:
            op = op.forwarded
            if op.is_device_op:
                srcs = op.args[1:] if isinstance(op, og.AssignOp) else \
                    (() if isinstance(op, og.Fill) else op.args)
                for a in srcs:
                    a = a.forwarded
                    if a.is_tensor_op:
                        readers.setdefault(_td(a).base, set()).add(op)
        for comp in self.computations:
            for v in comp.computation_op.values:
                v = v.forwarded
                if v.is_tensor_op:
                    returned.add(_td(v).base)
        return readers, returned

    def transform_ordered_ops(self, computation, ordered_ops, name):
        group = self.gpu_kernel_group(name)
        readers, returned = self._usage_maps()
        planner = FusionPlanner(self, fusion=self.fusion)
        for i, g in enumerate(planner.plan(ordered_ops, readers, returned)):
            if g.fusable:
                group.kernels.append(self.make_fused_kernel(g.ops, g.store_ops, "%s_k%d" % (name, i)))
            else:
                op = g.ops[0]
                if isinstance(op, og.ContiguousOp):
                    group.kernels.append(self.make_copy_kernel(op))
                elif isinstance(op, MomentsOp):
                    group.kernels.append(MomentsKernel(self, op))
                else:
                    raise ValueError("Unhandled op: {}".format(op))
        if self.chain_kernels and self.fusion:
            group.kernels = self._chained(group.kernels)
        self.kernel_groups[computation] = group
        computation.executor = group
        return name

    def _chained(self, kernels):
        """Runs of consecutive fused kernels with a reduction among them become KernelRuns."""
        out, run = [], []

        def flush():
            if len(run) >= 2 and (isinstance(run[0], MomentsKernel) or
                                  any(isinstance(op, og.ReductionOp) and op.reduction_axes.size > 1
                                      for k in run for op in k.ops)):
                out.append(KernelRun(self, run))
            else:
                out.extend(run)
            del run[:]

        for k in kernels:
            if type(k) is self.chain_member_class:
                run.append(k)
            elif type(k) is MomentsKernel:
                # (the statistics of rows and the kernels that use them may merge as well)
                flush()
                run.append(k)
            else:
                flush()
                out.append(k)
        flush()
        return out

    def make_fused_kernel(self, ops, store_ops, name):
        return FusedKernel(self, ops, store_ops, name)

    def make_copy_kernel(self, op):
        return CopyKernel(self, op)

    def finish_transform(self):
        pass

    def allocate_storage(self):
        pass

    def allocate(self):
        """Storage, initial values, and then -- where the reference compiles the kernels of every
        computation (float_ew2.py:1553-1653, at `initialize()`) -- the kernels are lowered and
        their programs asked for: compiled on the spot with jit=True, handed to the compile
        workers with jit="auto" (the computations start on the interpreter and pick the
        programs up when they are ready)."""
        if self.allocated:
            return
        super(HipTransformer, self).allocate()
        if self.jit is not False:
            for group in self.kernel_groups.values():
                group.bind()

    def close(self):
        for group in getattr(self, "kernel_groups", {}).values():
            if hasattr(group, "cancel_programs"):
                group.cancel_programs()
            if hasattr(group, "drop_graph") and getattr(self, "runtime", None) is not None:
                group.drop_graph()
        rt = getattr(self, "runtime", None)
        if rt is not None:
            try:
                rt.sync()
            except Exception:
                pass
            rt.close()
            self.runtime = None
