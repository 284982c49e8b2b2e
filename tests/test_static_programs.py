"""Host-side checks that need no GPU: the library loads and exports every
declared symbol, the generated program table is current, and graphs of the
benchmark patterns lower to specs the library maps onto a pre-built kernel."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.frontends import neon
from ngraph_hip.runtime import hiplib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ngraph_hip.h")).read()
    declared = set(re.findall(r"\b(ngh_[a-z0-9_]+)\s*\(", header))
    lib = hiplib.load_library()
    for name in sorted(declared):
        assert hasattr(lib, name), "libngraph_hip.so does not export %s" % name
    assert declared == set(hiplib.exported_symbols())


def test_generated_program_table_is_current():
    gen = os.path.join(ROOT, "ngraph-python_amd", "csrc", "gen_programs.py")
    assert subprocess.call([sys.executable, gen, "--check"]) == 0, \
        "csrc/ngh_programs.inc is stale: run gen_programs.py and rebuild"


def _kernels(t, f):
    t.initialize()
    out = []
    for k in t.kernel_groups[f].kernels:
        k.bind_buffers()
        for spec in getattr(k, "specs", []):
            out.append((k, spec))
    return out


def test_adam_lowers_to_one_streaming_kernel_with_a_prebuilt_program():
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    P = ng.make_axis(25600000, name="P")
    p, grad = ng.variable([P], initial_value=0.0), ng.placeholder([P])
    opt = neon.Adam()
    opt()
    updates, _, _ = opt.variable_update(p, grad)
    f = t.computation(updates, grad)
    big = [(k, s) for k, s in _kernels(t, f) if s.shape[0] > 1]
    assert len(big) == 1
    _, spec = big[0]
    assert spec.n_tensors == 5                  # m, g, v, ell, p: 4 reads + 3 writes per element
    plan = hiplib.plan_fused(spec, 0)
    assert plan["family"] == 0 and plan["V"] == 4 and plan["special"] >= 0
    t.close()


def test_batchnorm_lowering_recomputes_instead_of_materialising():
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", (256, 56, 56, 64)))
    x = ng.placeholder([C, H, W, N])
    gamma, beta = ng.variable([C], initial_value=1.0), ng.variable([C], initial_value=0.0)
    y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    f = t.computation([y, xmean, xvar], x)
    big = [s for _, s in _kernels(t, f) if s.shape[0] * s.shape[1] > 256]
    # no full-size intermediate is written: only the normalise kernel stores a big tensor
    stores_big = 0
    for s in big:
        for o in s.ops[:s.n_ops]:
            if o.opcode == hiplib.OPCODES["store"]:
                stores_big += 1
    assert stores_big == 1
    plan = hiplib.plan_fused(big[-1], 0)
    assert plan["V"] == 4 and plan["special"] >= 0
    t.close()


def test_spec_validation_rejects_malformed_programs():
    sb = hiplib.FusedSpecBuilder([16])
    t0 = sb.tensor(4096, [1])
    r = sb.reg()
    sb.emit("neg", r, r)                         # reads a register nothing defined
    sb.store(t0, r)
    spec = sb.build(compact=False)
    lib = hiplib.load_library()
    import ctypes
    assert lib.ngh_validate_fused(ctypes.byref(spec)) != 0
    assert b"undefined" in lib.ngh_last_error()
    sb = hiplib.FusedSpecBuilder([16, 4])
    t0, t1 = sb.tensor(4096, [4, 1]), sb.tensor(8192, [1, 0])
    sb.store(t1, sb.load(t0))                    # store through a broadcast view
    assert lib.ngh_validate_fused(ctypes.byref(sb.build())) != 0


def _hints(group):
    """{operand role string: cache hint} over the large specs of a bound kernel group."""
    out = []
    for k in group.kernels:
        for spec, uses in zip(getattr(k, "specs", []), getattr(k, "spec_uses", [])):
            for s, (base, is_read, is_written) in enumerate(uses):
                if int(np.prod(base.shape or (1,))) > 65536:
                    out.append((is_read, is_written, spec.tensors[s].cache_hint))
    return out


def test_cache_hints_adam_streams_loads_and_keeps_state_stores_cacheable():
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    P = ng.make_axis(1 << 20, name="P")
    p, grad = ng.variable([P], initial_value=0.0), ng.placeholder([P])
    opt = neon.Adam()
    opt()
    updates, _, _ = opt.variable_update(p, grad)
    f = t.computation(updates, grad)
    t.initialize()
    group = t.kernel_groups[f]
    group.bind()
    hints = _hints(group)
    assert len(hints) == 4                                        # p, g, m, v
    for is_read, is_written, hint in hints:
        assert is_read and hint & hiplib.NGH_CACHE_STREAM_LOAD    # each is read by this kernel only
        assert not hint & hiplib.NGH_CACHE_STREAM_STORE           # in-place state is read next step
    t.close()


def test_cache_hints_batchnorm_keeps_x_cacheable_and_streams_y():
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    t.chain_kernels = False       # (rows this short would merge into a row chain: the kernels are looked at one by one here)
    C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", (64, 16, 16, 16)))
    x = ng.placeholder([C, H, W, N])
    gamma, beta = ng.variable([C], initial_value=1.0), ng.variable([C], initial_value=0.0)
    y, xmean, xvar = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
    f = t.computation([y, xmean, xvar], x)
    t.initialize()
    group = t.kernel_groups[f]
    group.bind()
    moments = [k for k in group.kernels if type(k).__name__ == "MomentsKernel"]
    assert len(moments) == 1 and moments[0].x_cache_hint == 0     # x is read again by normalise
    hints = _hints(group)
    reads = [h for r, w, h in hints if r and not w]
    writes = [h for r, w, h in hints if w and not r]
    assert reads == [0]                                           # x: two readers, stays cacheable
    assert writes == [hiplib.NGH_CACHE_STREAM_STORE]              # y: a result nobody here reads
    t.close()


def test_cache_hints_of_a_row_chain_and_of_its_members():
    """A softmax merged into one chain: the chain is the only reader of x (its loads may stream)
    and nothing reads y again (its stores may stream); the three kernels it consists of, which
    run by themselves until the chain is compiled, read x one after the other, so none of them
    may stream it past the cache, and only the last writes a result nobody reads."""
    t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit=False)()
    N, C = ng.make_axis(4096, name="N"), ng.make_axis(1000, name="C")
    x = ng.placeholder([N, C])
    e = ng.exp((x - ng.max(x, out_axes=[N])) * 0.5)
    f = t.computation(e / ng.sum(e, out_axes=[N]), x)
    t.initialize()
    group = t.kernel_groups[f]
    group.bind()
    assert [type(k).__name__ for k in group.kernels] == ["ChainKernel"]
    chain = group.kernels[0]
    big = _hints(group)
    assert sorted(big) == [(False, True, hiplib.NGH_CACHE_STREAM_STORE), (True, False, hiplib.NGH_CACHE_STREAM_LOAD)]
    member_hints = []
    for m in chain.members:
        for spec, uses in zip(m.specs, m.spec_uses):
            for s, (base, is_read, is_written) in enumerate(uses):
                if int(np.prod(base.shape or (1,))) > 65536:
                    member_hints.append((is_read, is_written, spec.tensors[s].cache_hint))
    assert member_hints == [(True, False, 0), (True, False, 0), (True, False, 0),
                            (False, True, hiplib.NGH_CACHE_STREAM_STORE)]
    t.close()
