#!/usr/bin/env python
"""Benchmark of the fused elementwise / reduction / flex16 path on one MI355X.

The headline step is one pass of the batch-norm forward graph (statistics + normalise) over
x[256, 56, 56, 64] fp32 with inputs resident in HBM (configuration C2); the same run also
times the other two configurations of at least 64 MB, the Adam update over 25.6 M parameters
(C3) and the flex16 relu(x*w+b) over 16 M elements, 8 iterations a step (C5).  Prints ONE JSON
line: whole-job achieved HBM GB/s of C2 (algorithmic bytes / wall time per step), and per
configuration the step time over several blocks of steps (median, min, max), the roofline of
its dominant kernel from HIP-event timings taken in this run -- back to back ("warm": part of
the operands is still in the 256 MiB last-level cache from the launch before) and with that
cache displaced before every launch ("cold") -- and the NumPy oracle timed on the host cores as
the CPU baseline.  The two small configurations (C1, C4) are timed too, launch-bound as they are; `--compiled` adds five user
graphs on the interpreter and with kernels compiled at run time.
"""
from __future__ import print_function
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ngraph-python_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0
DISPLACE_BYTES = 512 << 20      # a device copy of this size between launches empties the last-level cache

# Bytes one launch requests from the memory side of L2, recorded with rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (each scaled by a device copy of known size) -- not measured by this run.  A figure
# is only reported for the very kernel and shape it was recorded on.
RECORDED_TRAFFIC = {
    ("C2", "special:batchnorm_k1/nt-stores", 51380224): (411167839, "profiles/c2_c3_c5_pmc_traffic.md"),
    ("C3", "special:adam_k1/nt-loads", 25600000): (716818595, "profiles/c2_c3_c5_pmc_traffic.md"),
    ("C5", "special:flex_relu_fma_k0", 16777216): (134547767, "profiles/c2_c3_c5_pmc_traffic.md"),
}


def recorded_traffic(config, kernel, elements):
    hit = RECORDED_TRAFFIC.get((config, kernel, elements))
    return {"traffic": hit[0] if hit else None,
            "traffic_source": ("requested bytes at L2 -> fabric, recorded in %s" % hit[1]) if hit else None}


# ------------------------------------------------------------------------------------- timing
def time_steps(rt, run, steps, warmup):
    for _ in range(warmup):
        run()
    rt.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    rt.sync()
    return (time.perf_counter() - t0) * 1e3 / steps


def step_blocks(rt, run, steps, warmup, blocks):
    """[ms per step] of `blocks` timed blocks of exactly `steps` steps; the first follows `warmup`
    untimed steps."""
    out = [time_steps(rt, run, steps, warmup)]
    for _ in range(blocks - 1):
        out.append(time_steps(rt, run, steps, 0))
    return out


def spread(ms):
    return {"blocks": len(ms), "median_ms": round(float(np.median(ms)), 5), "min_ms": round(min(ms), 5),
            "max_ms": round(max(ms), 5)}


class Displacer(object):
    """Empties the 256 MiB last-level cache between launches.

    dirty=False: a kernel reads 512 MiB (a sum), which leaves the cache full of clean lines: the
    next launch finds none of its operands there and has nothing else to wait for -- what a
    kernel meets when other kernels' inputs have passed through the cache since its operands
    were last touched.  dirty=True: a 512 MiB device-to-device copy, which also leaves up to
    256 MiB of freshly written lines that the memory system writes back while the next
    launch runs -- what a kernel meets right after a producer of other large results."""

    def __init__(self, rt, dirty=False):
        from ngraph_hip.runtime.hiplib import FusedSpecBuilder
        self.rt, self.dirty = rt, dirty
        self.a = rt.malloc(DISPLACE_BYTES)
        rt.memset32(self.a, 0, DISPLACE_BYTES // 4)
        if dirty:
            self.b = rt.malloc(DISPLACE_BYTES)
        else:
            self.b = rt.malloc(16)
            sb = FusedSpecBuilder([DISPLACE_BYTES // 4])
            src, dst = sb.tensor(self.a, [1]), sb.tensor(self.b, [0])
            sb.reduce("sum", sb.load(src), dst)
            self.spec = sb.build()
        rt.sync()

    def __call__(self):
        if self.dirty:
            self.rt.memcpy_d2d(self.b, self.a, DISPLACE_BYTES)
        else:
            self.rt.launch_fused(self.spec)

    def free(self):
        self.rt.free(self.a)
        self.rt.free(self.b)


def kernel_bytes(kernel):
    """Algorithmic bytes of one launch of a kernel: every operand once per direction."""
    if hasattr(kernel, "rows"):                         # the moments kernel reads x once, writes 3 floats a row
        return kernel.rows * kernel.R * 4 + kernel.rows * 12
    total = 0
    for spec in getattr(kernel, "specs", []):
        shape = [spec.shape[i] for i in range(3)]
        for i in range(spec.n_tensors):
            t = spec.tensors[i]
            n = 1
            for a in range(3):
                if t.strides[a] != 0:
                    n *= shape[a]
            loads = sum(1 for o in spec.ops[:spec.n_ops] if o.opcode == 1 and o.a == i)
            stores = sum(1 for o in spec.ops[:spec.n_ops] if o.opcode == 2 and o.dst == i)
            itemsize = {0: 4, 2: 4, 4: 4, 6: 1, 7: 1}.get(t.dtype, 2)
            total += n * itemsize * (min(loads, 1) + min(stores, 1))
    return total


def kernel_name(kernel):
    return "+".join(sum(kernel.describe(), [])) if hasattr(kernel, "describe") else type(kernel).__name__


def profile_kernels(group, rt, repeats, inner, displace=None):
    """Per kernel: algorithmic bytes and HIP-event duration per launch on the launch stream.
    Warm: `inner` launches back to back between one pair of events.  Cold (`displace` given):
    the cache is emptied before every launch, outside the event pair, one launch per pair."""
    out = []
    if displace is None:
        for k, times in group.profile(repeats=repeats, inner=inner):
            out.append({"kernel": kernel_name(k), "bytes": kernel_bytes(k), "ms": float(np.median(times))})
        return out
    for k in group.kernels:
        times = []
        for _ in range(repeats):
            displace()
            group.setup_kernel_execute(k)
            rt.timer_begin()
            k.execute()
            times.append(rt.timer_end())
            group.after_kernel_execute(k)
        out.append({"kernel": kernel_name(k), "bytes": kernel_bytes(k), "ms": float(np.median(times))})
    return out


def event_pair_overhead_ms(rt, repeats=20):
    """What a pair of events around nothing reads: the floor under every one-launch timing."""
    times = []
    for _ in range(repeats):
        rt.timer_begin()
        times.append(rt.timer_end())
    return float(np.median(times))


def cold_step_ms(group, rt, displace, repeats):
    times = []
    for _ in range(repeats):
        displace()
        rt.timer_begin()
        group()
        times.append(rt.timer_end())
    return float(np.median(times))


COLD_NOTE = ("one launch per event pair after a kernel has read 512 MiB, which leaves the last-level cache holding "
             "none of the operands and no dirty lines; the reading of an empty event pair is subtracted")


def roofline_of(config, kernels_warm, kernels_cold, elements, overhead=0.0):
    """Roofline block of the kernel with the longest warm duration."""
    i = max(range(len(kernels_warm)), key=lambda j: kernels_warm[j]["ms"])
    dom = kernels_warm[i]
    achieved = dom["bytes"] / (dom["ms"] * 1e-3) / 1e9
    out = {"bound": "hbm", "kernel": dom["kernel"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
           "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
           "algorithmic_bytes_per_launch": dom["bytes"], "avg_launch_ms": round(dom["ms"], 5),
           "timing": "HIP events on the launch stream, median over event pairs of 10 back-to-back launches"}
    out.update(recorded_traffic(config, dom["kernel"], elements))
    if kernels_cold:
        c = kernels_cold[i]
        ms = max(c["ms"] - overhead, 1e-6)
        cold = c["bytes"] / (ms * 1e-3) / 1e9
        out["cold"] = {"achieved": round(cold, 1), "frac": round(cold / HBM_PEAK_GBS, 4),
                       "avg_launch_ms": round(ms, 5), "timing": COLD_NOTE}
    return out


def config_block(name, workload, step_ms, nbytes, elems, kernels_warm, kernels_cold, cold_ms, roof_elems,
                 per_step=1, overhead=0.0, dirty_ms=None):
    ms = float(np.median(step_ms))
    if kernels_cold:
        kernels_cold = [dict(k, ms=max(k["ms"] - overhead, 1e-6)) for k in kernels_cold]
    blk = {"workload": workload, "ms_per_step": spread(step_ms),
           "GB/s": round(nbytes * per_step / (ms * 1e-3) / 1e9, 1),
           "frac_of_hbm_peak": round(nbytes * per_step / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "elements_per_s": round(elems * per_step / (ms * 1e-3), 1),
           "algorithmic_bytes_per_step": nbytes * per_step,
           "kernels": [dict({"kernel": k["kernel"], "ms": round(k["ms"], 5), "bytes": k["bytes"],
                             "GB/s": round(k["bytes"] / (k["ms"] * 1e-3) / 1e9, 1)},
                            **({"cold_ms": round(kernels_cold[i]["ms"], 5),
                                "cold_GB/s": round(k["bytes"] / (kernels_cold[i]["ms"] * 1e-3) / 1e9, 1)}
                               if kernels_cold else {}))
                       for i, k in enumerate(kernels_warm)],
           "roofline": roofline_of(name, kernels_warm, kernels_cold, roof_elems),
           "empty_event_pair_ms": round(overhead, 5)}

    def step(ms_):
        ms_ = max(ms_ - overhead, 1e-6)
        return {"ms": round(ms_, 5), "GB/s": round(nbytes / (ms_ * 1e-3) / 1e9, 1),
                "frac_of_hbm_peak": round(nbytes / (ms_ * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if cold_ms is not None:
        blk["cold_step"] = dict(step(cold_ms), timing="one step per event pair, " + COLD_NOTE[COLD_NOTE.index("after"):])
    if dirty_ms is not None:
        blk["step_after_a_512MiB_device_copy"] = dict(
            step(dirty_ms), timing="one step per event pair after a 512 MiB device-to-device copy: the step also "
                                   "waits for the write-back of the lines the copy left in the cache")
    return blk


# ------------------------------------------------------------------------------------- configurations
C2_DIMS = (256, 56, 56, 64)


def build_c2(ng, neon, t, dims, gamma_np, beta_np):
    C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", dims))
    x = ng.placeholder([C, H, W, N])
    gamma = ng.variable([C], initial_value=gamma_np)
    beta = ng.variable([C], initial_value=beta_np)
    y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    return t.computation([y, xmean, xvar], x), x


def bench_c2(ng, ngt, neon, workloads, args, want_cold, copy_calibration=0):
    dims = C2_DIMS
    n_elems = int(np.prod(dims))
    nbytes = 3 * n_elems * 4                                  # statistics read + normalise read + write
    t = ngt.make_transformer_factory("hipgpu")()
    rt = t.runtime
    x_np, gamma_np, beta_np = workloads.c2_inputs(dims[0], n_elems // dims[0], seed=1)
    f, x = build_c2(ng, neon, t, dims, gamma_np, beta_np)
    t.initialize()
    t.get_op_tensor_view(x)[...] = x_np.reshape(dims)        # inputs resident before timing
    group = t.kernel_groups[f]
    group()                                                    # binds buffers, first launch
    rt.sync()
    step_ms = step_blocks(rt, group, args.steps, args.warmup, args.blocks)
    warm = profile_kernels(group, rt, repeats=max(args.steps // 10, 5), inner=10)
    cold, cold_ms = None, None
    overhead = event_pair_overhead_ms(rt)
    dirty_ms = None
    if want_cold:
        d = Displacer(rt)
        cold = profile_kernels(group, rt, repeats=15, inner=1, displace=d)
        cold_ms = cold_step_ms(group, rt, d, 15)
        d.free()
        d = Displacer(rt, dirty=True)
        dirty_ms = cold_step_ms(group, rt, d, 15)
        d.free()
    if copy_calibration:
        y_view = t.get_op_tensor_view(f.computation_op.values[0])
        x_view = t.get_op_tensor_view(x)
        for _ in range(copy_calibration):
            rt.memcpy_d2d(y_view.ptr, x_view.ptr, n_elems * 4)
        rt.sync()
    group()
    rt.sync()
    # Parity at full size through a property that does not depend on it: per channel the
    # normalised output has mean beta and variance gamma^2 * var / (var + eps).  (The element by
    # element comparison with the oracle at this size is tests/test_full_size_gpu.py.)
    y = t.get_op_tensor_view(f.computation_op.values[0]).get(None).reshape(dims[0], -1).astype(np.float64)
    var = x_np.astype(np.float64).var(axis=1)
    g64, b64 = gamma_np.astype(np.float64), beta_np.astype(np.float64)
    assert np.abs(y.mean(axis=1) - b64).max() < 1e-4, "normalised output: per-channel mean is not beta"
    assert np.abs(y.var(axis=1) - g64 * g64 * var / (var + 1e-5)).max() < 1e-3, \
        "normalised output: per-channel variance is not gamma^2 var / (var + eps)"
    boundary = call_boundary(t, f, x, x_np.reshape(dims))
    t.close()
    workload = ("C2 batch-norm forward: x fp32 [256,56,56,64] ~N(0.5,2), gamma, beta ~U(0.5,1.5), statistics over "
                "H,W,N then normalise; algorithmic bytes 616562688 per step")
    blk = config_block("C2", workload, step_ms, nbytes, n_elems, warm, cold, cold_ms, n_elems, overhead=overhead,
                       dirty_ms=dirty_ms)
    blk["call_boundary"] = boundary
    return blk, x_np, gamma_np, beta_np


def call_boundary(t, f, x, x_host, repeats=5):
    """What a caller of Computation.__call__ sees, with NumPy arrays in pageable host memory on
    both sides (never `value`, which has its inputs resident): the whole call, and its two
    transfers alone -- x written through its device tensor, y read back into a fresh array."""
    x_view = t.get_op_tensor_view(x)
    y_view = t.get_op_tensor_view(f.computation_op.values[0])
    n = x_host.nbytes
    call, put, get = [], [], []
    for _ in range(repeats):
        t0 = time.perf_counter()
        f(x_host)
        call.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        x_view[...] = x_host
        put.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        y = y_view.get(None)
        get.append(time.perf_counter() - t0)
        del y
    med = lambda v: float(np.median(v))
    return {"call_ms": round(med(call) * 1e3, 3), "host_to_device_ms": round(med(put) * 1e3, 3),
            "host_to_device_GB/s": round(n / med(put) / 1e9, 1), "device_to_host_ms": round(med(get) * 1e3, 3),
            "device_to_host_GB/s": round(n / med(get) / 1e9, 1), "bytes_each_way": n,
            "what": "Computation.__call__ with x and y as NumPy arrays in pageable memory: x in, the step, y and "
                    "the statistics out; large copies go through the context's pinned staging buffers"}


def bench_c3(ng, ngt, neon, workloads, args, want_cold):
    n = 25600000
    t = ngt.make_transformer_factory("hipgpu")()
    rt = t.runtime
    p_np, g_np, _, _ = workloads.c3_inputs(n)
    P = ng.make_axis(n, name="P")
    p, grad = ng.variable([P], initial_value=p_np), ng.placeholder([P])
    opt = neon.Adam()
    opt()
    updates, _, _ = opt.variable_update(p, grad)
    f = t.computation(updates, grad)
    f(g_np)                                   # the warm step (t = 1); inputs stay resident
    group = t.kernel_groups[f]
    steps = max(args.steps // 2, 5)
    step_ms = step_blocks(rt, group, steps, args.warmup, args.blocks)
    warm = profile_kernels(group, rt, repeats=max(steps // 10, 5), inner=10)
    cold, cold_ms, dirty_ms = None, None, None
    overhead = event_pair_overhead_ms(rt)
    if want_cold:
        d = Displacer(rt)
        cold = profile_kernels(group, rt, repeats=15, inner=1, displace=d)
        cold_ms = cold_step_ms(group, rt, d, 15)
        d.free()
        d = Displacer(rt, dirty=True)
        dirty_ms = cold_step_ms(group, rt, d, 15)
        d.free()
    t.close()
    workload = ("C3 Adam update in place over 25.6 M fp32 parameters (p, m, v read and written, grad read): "
                "algorithmic bytes 716800000 per step; timed from step 2 on")
    return config_block("C3", workload, step_ms, 716800000, n, warm, cold, cold_ms, n, overhead=overhead,
                        dirty_ms=dirty_ms)


class _Times(object):
    """A kernel group whose step is `n` runs of another group (C5: 8 iterations a step)."""

    def __init__(self, group, n):
        self.group, self.n, self.kernels = group, n, group.kernels

    def __call__(self):
        for _ in range(self.n):
            self.group()


def bench_c5(ng, ngt, neon, workloads, args, want_cold):
    n = 16 * 1024 * 1024
    t = ngt.make_transformer_factory("flexhip")()
    rt = t.runtime
    x_np, w_np, b_np = workloads.c5_inputs(n)
    P = ng.make_axis(n, name="P")
    x, w, b = ng.placeholder([P]), ng.placeholder([P]), ng.placeholder([P])
    f = t.computation(neon.rectlin(x * w + b), x, w, b)
    f(x_np, w_np, b_np)
    group = t.kernel_groups[f]
    group()
    rt.sync()
    eight = _Times(group, 8)
    steps = max(args.steps // 4, 5)
    step_ms = step_blocks(rt, eight, steps, args.warmup, args.blocks)
    # the kernel as it runs inside a step: 8 iterations between one pair of events
    times = []
    for _ in range(max(steps // 5, 5)):
        rt.timer_begin()
        eight()
        times.append(rt.timer_end() / 8)
    name = "+".join(kernel_name(k) for k in group.kernels)
    warm = [{"kernel": name, "bytes": 134217728, "ms": float(np.median(times))}]
    cold, cold_ms = None, None
    overhead = event_pair_overhead_ms(rt)
    if want_cold:
        d = Displacer(rt)
        times = []
        for _ in range(15):
            d()
            rt.timer_begin()
            group()
            times.append(rt.timer_end())
        cold = [{"kernel": name, "bytes": 134217728, "ms": float(np.median(times))}]
        d.free()
    mode = "device-resident" if t.flex_manager.resident else "host-managed"
    t.close()
    workload = ("C5 flex16 y = relu(x*w+b) over 16777216 elements, int16 mantissas with per-tensor exponents, "
                "max|mantissa| feeding the exponent update, 8 iterations per step (%s exponent management, the "
                "default of the flexhip transformer); algorithmic bytes 134217728 per iteration" % mode)
    blk = config_block("C5", workload, step_ms, 134217728, n, warm, cold, cold_ms, n, per_step=8, overhead=overhead)
    blk["flex16_elements_per_s"] = blk["elements_per_s"]
    return blk


def small_configs(ng, ngt, neon, workloads, steps, warmup):
    """C1 (8 MB) and C4 (1.8 MB) with inputs resident.  At these sizes a launch takes longer than
    its memory traffic: the blocks carry the step time, every kernel's duration from HIP events,
    and a roofline block marked as bound by launch latency (the HBM fraction is reported, but is
    not what limits these two)."""
    out = {}

    def run(name, workload, t, f, nbytes, elems):
        group = t.kernel_groups[f]
        group()
        t.runtime.sync()
        ms = step_blocks(t.runtime, group, steps, warmup, 3)
        kern = profile_kernels(group, t.runtime, repeats=5, inner=10)
        blk = config_block(name, workload, ms, nbytes, elems, kern, None, None, elems)
        blk["roofline"]["bound"] = "launch"
        # (two kernels that depend on nothing of each other go to the device as one launch when the
        # library has them built as a pair: the kernel group knows after its first executions)
        paired = len(getattr(group, "_pairs", None) or ())
        blk["roofline"]["note"] = ("%d kernel(s) in %d launch(es) per step; run one by one the kernels take %.1f us, "
                                   "the step takes %.1f us; at 8 TB/s the step's %d bytes would take %.2f us" %
                                   (len(kern), len(kern) - paired, sum(k["ms"] for k in kern) * 1e3,
                                    float(np.median(ms)) * 1e3, nbytes, nbytes / 8e12 * 1e6))
        out[name] = blk
        t.close()

    t = ngt.make_transformer_factory("hipgpu")()
    x_np, a, b = workloads.c1_inputs((1024, 1024))
    H, W = ng.make_axis(1024, name="H"), ng.make_axis(1024, name="W")
    x, pa, pb = ng.placeholder([H, W]), ng.placeholder(()), ng.placeholder(())
    f = t.computation(ng.tanh(pa * x + pb) * ng.sigmoid(x), x, pa, pb)
    f(x_np, a, b)
    run("C1", "C1 y = tanh(a*x+b)*sigmoid(x), x fp32 [1024,1024] ~N(0,1), a, b ~U(-1,1): one fused kernel; "
        "algorithmic bytes 8388608 per step", t, f, 8388608, 1048576)
    t = ngt.make_transformer_factory("hipgpu")()
    Hn, Nn = 1024, 64
    gates_np, cprev_np = workloads.c4_inputs(Hn, Nn)
    H, N, G = ng.make_axis(Hn, name="H"), ng.make_axis(Nn, name="N"), ng.make_axis(4 * Hn, name="G")
    gates_st, cprev_st = ng.placeholder([N, G]), ng.placeholder([N, H])
    gates, c_prev = ng.axes_with_order(gates_st, [G, N]), ng.axes_with_order(cprev_st, [H, N])
    parts = {k: ng.cast_axes(ng.tensor_slice(gates, [slice(j * Hn, (j + 1) * Hn), slice(None)]), [H, N])
             for j, k in enumerate(("i", "f", "o", "g"))}
    h, c = neon.lstm_cell(parts, c_prev, H, None)
    f = t.computation([c, h, ng.sum(gates, out_axes=[G])], gates_st, cprev_st)
    f(gates_np, cprev_np)
    run("C4", "C4 LSTM cell on transposed storage: gates fp32 [4H,N], c_prev [H,N], H=1024, N=64; c, h and the "
        "bias gradient sum over N; algorithmic bytes 1851392 per step", t, f, 1851392, 327680)
    return out


# ------------------------------------------------------------------------------------- user graphs
def user_graphs(ng, An=8192, Bn=8192):
    """(name, results, inputs, passes over an An x Bn fp32 tensor) of graphs the library has no
    built-in program for: what a user's own elementwise / reduction code looks like."""
    A, B = ng.make_axis(An, name="A"), ng.make_axis(Bn, name="B")
    x, y, w = ng.placeholder([A, B]), ng.placeholder([A, B]), ng.placeholder([A, B])
    z = ng.tanh(x * y + 0.5) / (ng.absolute(y) + 1.0)
    yield "chain_3in_2out", [z * w, ng.maximum(z, w) - x], [x, y, w], 5
    yield "gelu_tanh_form", [0.5 * x * (1.0 + ng.tanh(0.79788456 * (x + 0.044715 * x * x * x)))], [x], 2
    yield "chain_with_column_max", [z, ng.max(z, out_axes=[B])], [x, y], 3
    yield "row_sum_of_squared_difference", [ng.sum(ng.square(x - y), out_axes=[A])], [x, y], 2
    e = ng.exp(x - ng.max(x, out_axes=[A]))
    # (three kernels read x three times; merged into one row-chain kernel they read it once)
    yield "softmax_rows", [e / ng.sum(e, out_axes=[A])], [x], {"chain": 2, "kernels": 4}


def compiled_vs_interpreted(ng, ngt, steps, warmup, An=8192, Bn=8192):
    """The same computations with the transformer's default kernel choice (programs compiled at
    run time for large stages), on the interpreter alone (jit=False) and with compilation
    forced for every stage (jit=True): ms per step, algorithmic GB/s, kernels."""
    out = {}
    for name, results, inputs, passes in user_graphs(ng, An, Bn):
        row = {}
        # (interpreter first: a compiled program, once loaded, serves every transformer of the process)
        for label, mode in (("interpreted", False), ("default", None), ("compiled", True)):
            t = ngt.make_transformer_factory("hipgpu", jit=mode)()
            try:
                f = t.computation(results, *inputs)
                f(*[np.random.RandomState(1 + i).uniform(-1, 1, p.axes.lengths).astype(np.float32)
                    for i, p in enumerate(inputs)])
                group = t.kernel_groups[f]
                if hasattr(group, "wait_for_programs"):
                    group.wait_for_programs()
                group()
                t.runtime.sync()
                ms = float(np.median(step_blocks(t.runtime, group, steps, warmup, 3)))
                names = [d for k in group.kernels for ds in k.describe() for d in ds]
                n_passes = passes if not isinstance(passes, dict) else \
                    passes["chain" if any("/chain-of-" in d for d in names) else "kernels"]
                nbytes = n_passes * An * Bn * 4
                row[label] = {
                    "passes": n_passes,
                    "ms_per_step": round(ms, 5), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "kernels": [d for k in group.kernels for ds in k.describe() for d in ds]}
                if label != "interpreted":
                    # one step per event pair with the cache emptied by a 512 MiB read before it
                    d = Displacer(t.runtime)
                    cold = max(cold_step_ms(group, t.runtime, d, 9) - event_pair_overhead_ms(t.runtime), 1e-6)
                    d.free()
                    row[label]["cold_step"] = {"ms": round(cold, 5), "GB/s": round(nbytes / (cold * 1e-3) / 1e9, 1),
                                               "frac_of_hbm_peak": round(nbytes / (cold * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
            finally:
                t.close()
        row["first_run"] = first_run_latency(name)
        out[name] = row
    return out


def first_run_latency(name):
    """What a machine pays once per program, measured in a child process (in this one the
    programs are loaded already): seconds `initialize()` of a transformer with jit=True takes
    with an empty program cache, hipcc compiling every stage's program."""
    import subprocess
    report = {}
    for compiler in ("hipcc", "hiprtc"):          # a subprocess per program / inside the process
        try:
            out = subprocess.run([sys.executable, os.path.abspath(__file__), "--first-run-of", name],
                                 stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600,
                                 env=dict(os.environ, NGH_JIT_COMPILER=compiler, AMD_COMGR_CACHE="0"))
            # (without the compiler library's own cache of results: this process has compiled the
            # same source a moment ago)
            report[compiler] = json.loads(out.stdout.decode().strip().splitlines()[-1])
        except Exception as e:
            report[compiler] = {"error": str(e)[:200]}
    return report


def first_run_child(name):
    """The child of first_run_latency: one JSON line."""
    import shutil
    import tempfile
    import ngraph_hip as ng
    import ngraph_hip.transformers as ngt
    tmp = tempfile.mkdtemp(prefix="ngh_programs_")
    os.environ["NGH_PROGRAM_CACHE"] = tmp
    try:
        results, inputs = [(r, i) for n, r, i, _ in user_graphs(ng) if n == name][0]
        seconds = {}
        for label, mode in (("lowering_only_s", False), ("initialize_s_empty_cache", True)):
            t = ngt.make_transformer_factory("hipgpu", jit=mode)()
            try:
                t.computation(results, *inputs)
                t0 = time.perf_counter()
                t.initialize()
                seconds[label] = round(time.perf_counter() - t0, 3)
            finally:
                t.close()
        n = len([f for f in os.listdir(tmp) if f.endswith(".so") or f.endswith(".ngco")])
        seconds.update({"programs": n, "what": "jit=True: every stage's program compiled at initialize() with the "
                        "compiler NGH_JIT_COMPILER names (hipcc: subprocesses, up to 4 at a time; hiprtc: inside "
                        "the process, every variant of a program's kernels in one compilation); a later process "
                        "finds the libraries in the cache"})
        print(json.dumps(seconds))
    except Exception as e:                      # no hipcc on this machine
        print(json.dumps({"error": str(e)[:200]}))
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


# ------------------------------------------------------------------------------------- shapes
def shape_survey_cases(ng):
    """(name, results, inputs, algorithmic bytes) of graphs over 64-270 MB tensors in the layouts
    and extents that everyday graphs have: broadcasts, transposed operands, reductions along,
    across and over several axes, many short rows, odd extents."""
    def ax(n, name):
        return ng.make_axis(n, name=name)
    A, B = ax(8192, "A"), ax(8192, "B")
    x, y = ng.placeholder([A, B]), ng.placeholder([A, B])
    row_vec, col_vec = ng.placeholder([B]), ng.placeholder([A])
    full = 8192 * 8192 * 4
    yield "x + b[B] (operand broadcast along rows)", [x + row_vec], [x, row_vec], 2 * full
    yield "x * c[A] (operand broadcast along the contiguous axis)", [x * col_vec], [x, col_vec], 2 * full
    xt = ng.placeholder([B, A])
    yield "tanh(transposed x) * y", [ng.tanh(ng.axes_with_order(xt, [A, B])) * y], [xt, y], 3 * full
    yield "sum across the contiguous axis [8192,8192]", [ng.sum(x, out_axes=[B])], [x], full
    yield "sum along the contiguous axis [8192,8192]", [ng.sum(x, out_axes=[A])], [x], full
    N, C, HW = ax(64, "N"), ax(256, "C"), ax(3136, "HW")
    v = ng.placeholder([N, C, HW])
    nchw = 64 * 256 * 3136 * 4
    yield "[N,C,HW] sum over N and HW", [ng.sum(v, out_axes=[C])], [v], nchw
    yield "[N,C,HW] sum over C", [ng.sum(v, out_axes=[N, HW])], [v], nchw
    yield "[N,C,HW] sum over HW", [ng.sum(v, out_axes=[N, C])], [v], nchw
    gamma, beta = ng.placeholder([C]), ng.placeholder([C])
    mean, var = ng.mean(v, out_axes=[C]), ng.variance(v, out_axes=[C])
    yield ("[N,C,HW] batch norm (statistics over N and HW, normalise; 3 passes)",
           [gamma * ((v - mean) * ng.reciprocal(ng.sqrt(var + 1e-5))) + beta], [v, gamma, beta], 3 * nchw)
    for rows, k in ((131072, 256), (32768, 1024), (32768, 1000), (32768, 1001), (8192, 4096)):
        R, K = ax(rows, "R%d" % k), ax(k, "K%d" % k)
        w = ng.placeholder([R, K])
        mu, vv = ng.mean(w, out_axes=[R]), ng.variance(w, out_axes=[R])
        # (as one row-chain kernel x is read once; else the one-pass moments kernel reads it, then
        # the normalise kernel)
        yield ("layer norm of rows [%d,%d] (statistics, normalise)" % (rows, k),
               [(w - mu) * ng.reciprocal(ng.sqrt(vv + 1e-5))], [w],
               {"chain": 2 * rows * k * 4, "kernels": 3 * rows * k * 4})
        e = ng.exp(w - ng.max(w, out_axes=[R]))
        # (as one row-chain kernel the operand is read once and the result written once; as three
        # kernels it is read three times)
        yield ("softmax of rows [%d,%d] (maximum, sum of exponentials, normalise)" % (rows, k),
               [e / ng.sum(e, out_axes=[R])], [w], {"chain": 2 * rows * k * 4, "kernels": 4 * rows * k * 4})
    # the same softmax with flex16 storage (the flexhip transformer): the maximum, the sum and the
    # result are flex16 tensors with an exponent each; 2 bytes per element either way
    for rows, k in ((32768, 1024), (32768, 1000)):
        R, K = ax(rows, "FR%d" % k), ax(k, "FK%d" % k)
        w = ng.placeholder([R, K])
        e = ng.exp(w - ng.max(w, out_axes=[R]))
        yield ("flex16 softmax of rows [%d,%d] (maximum, sum of exponentials, normalise)" % (rows, k),
               [e / ng.sum(e, out_axes=[R])], [w],
               {"chain": 2 * rows * k * 2, "kernels": 4 * rows * k * 2, "transformer": "flexhip"})
    # classes x samples, the layout of the neon front end (op_graph.py:3849): the reduced axis is the
    # strided one; as one column-chain kernel the operand is read once (few classes: kept in
    # registers) or re-read from the caches by the later stages
    for classes, samples in ((1000, 32768), (10, 4194304), (100, 327680)):
        K, S = ax(classes, "KC%d" % classes), ax(samples, "SC%d" % classes)
        w = ng.placeholder([K, S])
        e = ng.exp(w - ng.max(w, out_axes=[S]))
        yield ("softmax over classes [%d,%d] (classes x samples: the reduced axis strided)" % (classes, samples),
               [e / ng.sum(e, out_axes=[S])], [w],
               {"chain": 2 * classes * samples * 4, "kernels": 4 * classes * samples * 4})
    O1, O2 = ax(8191, "O1"), ax(8191, "O2")
    o, o2 = ng.placeholder([O1, O2]), ng.placeholder([O1, O2])
    odd = 8191 * 8191 * 4
    yield "tanh(x * y) [8191,8191]", [ng.tanh(o * o2)], [o, o2], 3 * odd
    yield "sum along the contiguous axis [8191,8191]", [ng.sum(o, out_axes=[O1])], [o], odd
    yield "sum across the contiguous axis [8191,8191]", [ng.sum(o, out_axes=[O2])], [o], odd


def shape_survey(ng, ngt, steps, warmup, only=""):
    """The graphs of shape_survey_cases with the transformer's default kernel choice (programs
    compiled at run time loaded before timing): ms per step, algorithmic GB/s, and each
    kernel's duration from HIP events."""
    out = {}
    for name, results, inputs, nbytes in shape_survey_cases(ng):
        if only and only not in name:
            continue
        t = ngt.make_transformer_factory(nbytes.get("transformer", "hipgpu") if isinstance(nbytes, dict) else "hipgpu")()
        try:
            f = t.computation(results, *inputs)
            values = [np.random.RandomState(i).uniform(0.5, 1.5, p.axes.lengths).astype(np.float32)
                      for i, p in enumerate(inputs)]
            f(*values)
            group = t.kernel_groups[f]
            f(*values)                                   # the second run starts the compile workers
            error = group.wait_for_programs()
            group()
            t.runtime.sync()
            ms = float(np.median(step_blocks(t.runtime, group, steps, warmup, 3)))
            kernels = [("+".join(sorted(set(d for ds in k.describe() for d in ds))), round(float(np.median(times)) * 1e3, 1))
                       for k, times in group.profile(repeats=3, inner=10)]
            if isinstance(nbytes, dict):
                chained = any("chain-of-" in d for d, _ in kernels)
                passes = nbytes["kernels"] // (nbytes["chain"] // 2)
                nbytes = nbytes["chain" if chained else "kernels"]
                name += " (one chain kernel; 2 passes)" if chained else \
                    " (%d kernels; %d passes)" % (len(kernels), passes)
            out[name] = {"ms_per_step": round(ms, 5), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                         "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                         "algorithmic_bytes_per_step": int(nbytes),
                         "kernels_us": kernels}
            if error:
                out[name]["compiler"] = error
        finally:
            t.close()
    return out


# ------------------------------------------------------------------------------------- CPU baseline
def cpu_baseline_c2(configs, x, gamma, beta, budget_s=20.0):
    ws = configs.Workspace()
    configs.c2_cpu(x, gamma, beta, ws=ws)                       # warm, allocates the pools
    times, t_start = [], time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        configs.c2_cpu(x, gamma, beta, ws=ws)
        times.append(time.perf_counter() - t0)
    sec = float(np.median(times))
    return {"value": round(616562688 / sec / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "full C2 workload, %d runs, median %.3f s/step; NumPy %s ufuncs are "
                      "single-threaded (host has %d cpus)" % (len(times), sec, np.__version__,
                                                             os.cpu_count())}


def cpu_baseline_others(configs, budget_s=4.0):
    """C3 and C5 on the host: a few runs each (bounded), in the unit of their configuration."""
    out = {}
    n = 25600000
    p, g, m, v = configs.c3_inputs(n)
    ws = configs.Workspace()
    configs.c3_cpu(p, g, m, v, 1, ws=ws)
    times, t_start, step = [], time.perf_counter(), 2
    while len(times) < 2 or (time.perf_counter() - t_start < budget_s and len(times) < 10):
        t0 = time.perf_counter()
        configs.c3_cpu(p, g, m, v, step, ws=ws)
        times.append(time.perf_counter() - t0)
        step += 1
    sec = float(np.median(times))
    out["C3"] = {"value": round(716800000 / sec / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                 "sample": "full C3 step, %d runs, median %.3f s" % (len(times), sec)}
    from oracle import flex_model as fm
    n = 16 * 1024 * 1024
    x, w, b = configs.c5_inputs(n)
    tx, tw, tb, ty = (fm._SimTensor((n,)) for _ in range(4))
    tx.host_write(x)
    tw.host_write(w)
    tb.host_write(b)
    ws = configs.Workspace()
    times, t_start = [], time.perf_counter()
    while len(times) < 2 or (time.perf_counter() - t_start < budget_s and len(times) < 8):
        t0 = time.perf_counter()
        ty.kernel_write(lambda: configs.c5_cpu_float(tx.load(), tw.load(), tb.load(), ws=ws))
        times.append(time.perf_counter() - t0)
    sec = float(np.median(times))
    out["C5"] = {"value": round(n / sec, 1), "unit": "flex16 elements/s", "cores": 1, "kind": "port",
                 "sample": "one C5 iteration (dequantise, relu(x*w+b), quantise, max|mantissa|, exponent "
                           "policy) of the NumPy flex model, %d runs, median %.3f s" % (len(times), sec)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=5,
                    help="timed blocks of --steps steps (the first gives the headline, all give the spread)")
    ap.add_argument("--configs", default="c2,c3,c5", help="which of c2, c3, c5 to run (c2 always runs)")
    ap.add_argument("--no-cold", action="store_true", help="skip the measurements with a displaced cache")
    ap.add_argument("--all", action="store_true", help="(kept for old command lines: C1 and C4 are always timed)")
    ap.add_argument("--compiled", action="store_true",
                    help="also time five user graphs: default kernel choice, interpreter only, compiled "
                         "(needs hipcc unless the program cache already holds them)")
    ap.add_argument("--first-run-of", default="", help=argparse.SUPPRESS)
    ap.add_argument("--only", default="", help="with --shapes: only the cases whose name contains this text")
    ap.add_argument("--shapes", action="store_true",
                    help="also time a survey of everyday layouts and extents (broadcasts, transposed operands, "
                         "reductions over one and several axes, many short rows, odd extents)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="N",
                    help="also issue N device-to-device copies of x (205 520 896 bytes each): a "
                         "kernel of known traffic to scale rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (--gpus 1); the path shards without "
              "exchange except for tiny statistics all-reduces, which are not part of this run.",
              file=sys.stderr)
        sys.exit(2)
    args.blocks = max(1, args.blocks)
    if args.first_run_of:
        first_run_child(args.first_run_of)
        return
    which = set(s.strip().lower() for s in args.configs.split(","))

    import ngraph_hip as ng
    import ngraph_hip.transformers as ngt
    from ngraph_hip.frontends import neon
    from ngraph_hip.testing import workloads

    c2, x_np, gamma_np, beta_np = bench_c2(ng, ngt, neon, workloads, args, not args.no_cold, args.copy_calibration)
    ms = c2["ms_per_step"]["median_ms"]
    value = c2["algorithmic_bytes_per_step"] / (ms * 1e-3) / 1e9
    out = {"metric": "achieved HBM GB/s on fused elementwise/reduction graphs (batch-norm forward); flex16 elem/s "
                     "under configs.C5",
           "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": c2["workload"], "elements": int(np.prod(C2_DIMS)),
                      "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                      "elements_per_s": c2["elements_per_s"], "kernels": c2["kernels"],
                      "ms_per_step_blocks": c2["ms_per_step"],
                      "value_is": "median over %d blocks of %d back-to-back steps each" % (args.blocks, args.steps)},
           "roofline": c2["roofline"]}
    if "cold_step" in c2:
        out["config"]["cold_step"] = c2["cold_step"]
    out["configs"] = {"C2": c2}
    if "c3" in which:
        out["configs"]["C3"] = bench_c3(ng, ngt, neon, workloads, args, not args.no_cold)
    if "c5" in which:
        out["configs"]["C5"] = bench_c5(ng, ngt, neon, workloads, args, not args.no_cold)
    out["configs"].update(small_configs(ng, ngt, neon, workloads, max(5, args.steps // 4), 2))
    if args.shapes:
        out["shapes"] = shape_survey(ng, ngt, max(20, args.steps // 4), 2, args.only)
    if args.compiled:
        out["compiled_at_run_time"] = compiled_vs_interpreted(ng, ngt, max(20, args.steps // 4), 2)
    if not args.no_cpu:
        # the only leg that needs the test oracle: its NumPy statements are what is timed
        from oracle import configs
        out["cpu_baseline"] = cpu_baseline_c2(configs, x_np, gamma_np, beta_np)
        others = cpu_baseline_others(configs)
        for name, blk in others.items():
            if name in out["configs"]:
                out["configs"][name]["cpu_baseline"] = blk
    print(json.dumps(out))


if __name__ == "__main__":
    main()
