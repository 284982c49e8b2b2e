"""Run-time compiled programs: a computation's stages that the library has no compiled kernel for
are written out as program tables, compiled by hipcc and loaded (the reference's counterpart is
the NVRTC compilation of generated CUDA C, float_ew2.py:1553-1653).  A compiled program must give
what the interpreter gives for the same spec, to the last bit (same skeleton, same op
definitions, same order of operations)."""
import ctypes
import os

import numpy as np
import pytest

import ngraph_hip as ng
import ngraph_hip.transformers as ngt
from ngraph_hip.runtime import hiplib, jit
from conftest import default_kernel_choice

import jit_cases


def _dry_kernels(case, backend="hipgpu"):
    t = ngt.make_transformer_factory(backend, dry_run=True)()
    results, inputs = case()
    f = t.computation(results, *inputs)
    t.initialize()
    kernels = t.kernel_groups[f].kernels
    for k in kernels:
        k.bind_buffers()
    return t, kernels


def test_uncovered_programs_are_found_and_rendered():
    t, kernels = _dry_kernels(jit_cases.case_elementwise)
    try:
        programs = jit.uncovered_programs(kernels, "case")
        assert len(programs) == 1 and programs[0][8] == 0          # one streaming elementwise stage
        text = jit.source_text(programs)
        assert 'extern "C" int ngh_program_library' in text and "launch_static<LP_%s_0>" % programs[0][0] in text
        # a built-in program is not compiled again
        t2, k2 = _dry_kernels(lambda: (lambda x: ([ng.sum(x, out_axes=[x.axes[0]])], [x]))(
            ng.placeholder([ng.make_axis(4096, name="A"), ng.make_axis(4096, name="B")])))
        try:
            assert jit.uncovered_programs(k2, "sum") == []
        finally:
            t2.close()
    finally:
        t.close()


def test_program_library_compiles_and_checks_its_caller(tmp_path, monkeypatch):
    """hipcc cross-compiles a program library without a device; its entry point refuses a caller
    built from other sources (ABI number, structure sizes)."""
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    monkeypatch.setenv("NGH_JIT_COMPILER", "hipcc")
    t, kernels = _dry_kernels(jit_cases.case_row_reduction_with_store)
    try:
        programs = jit.uncovered_programs(kernels, "case")
        assert programs
        path = jit.compile_programs(programs)
        assert os.path.dirname(path) == str(tmp_path)
        assert jit.compile_programs(programs) == path                  # second time: from the cache
        lib = ctypes.CDLL(path)
        fn = lib.ngh_program_library
        fn.argtypes = [ctypes.c_int, ctypes.c_uint, ctypes.c_uint, ctypes.POINTER(ctypes.c_void_p)]
        out = ctypes.c_void_p()
        assert fn(hiplib.NGH_ABI_VERSION + 1, 0, 0, ctypes.byref(out)) == -1
        assert fn(hiplib.NGH_ABI_VERSION, 1, 1, ctypes.byref(out)) == -1
    finally:
        t.close()


@pytest.mark.parametrize("compiler", ["hipcc", "hiprtc"])
def test_every_case_compiles_for_gfx950(compiler, monkeypatch):
    """Every skeleton's generated source compiles, with hipcc (which cross-compiles without a
    device) into shared objects and with hiprtc, inside the process, into code bundles.  The
    libraries land in the program cache, where the GPU tests of this file find them."""
    monkeypatch.setenv("NGH_JIT_COMPILER", compiler)
    paths = jit_cases.precompile()
    assert len(paths) >= 40 and all(os.path.exists(p) for p in paths)
    assert all(p.endswith(".so" if compiler == "hipcc" else ".ngco") for p in paths)


def test_kernel_names_of_a_program_description():
    """ngh_program_kernels: which kernels a program may launch follows from its description alone
    (no device): cache-policy variants, ragged-row forms only where the program allows them,
    non-temporal-store variants only where it stores, the stages of a chain in its kernels' names."""
    from ngraph_hip.runtime import hiplib
    load, store, add, rsum = (hiplib.OPCODES[n] for n in ("load", "store", "add", "sum"))
    ew = {"name": "jit_a", "type_name": "LP_a_0", "family": 0, "V": 4, "n_stat_slots": 0,
          "ops": [[load, 0, 0, 0], [load, 1, 1, 0], [add, 0, 0, 1], [store, 2, 0, 0]],
          "dtypes": [0, 0, 0], "bcast": [0, 0, 0], "rowshared": [0, 0, 0], "staged": [-1, -1, -1], "red_out": []}
    names = hiplib.program_kernels(hiplib.program_descs([ew]), 0)
    assert names[0] == "ngh::ew_static_kernel<ngh::LP_a_0, 0>" and names[3].endswith(", 3>")
    assert names[4] == "ngh::ew_ragged_static_kernel<ngh::LP_a_0, 0>" and not any(names[8:])
    flex = dict(ew, dtypes=[1, 1, 1], n_stat_slots=1)          # flex16: no ragged rows, deferred statistics
    names = hiplib.program_kernels(hiplib.program_descs([flex]), 0)
    assert not any(names[4:8]) and names[8] == "ngh::ew_static_lazy_kernel<ngh::LP_a_0, 0>"
    row_sum = {"name": "jit_b", "type_name": "LP_b_0", "family": 1, "V": 4, "n_stat_slots": 0,
               "ops": [[load, 0, 0, 0], [rsum, 0, 0, 0]], "dtypes": [0, 0], "bcast": [0, 1], "rowshared": [0, 0],
               "staged": [-1, -1], "red_out": [1]}
    names = hiplib.program_kernels(hiplib.program_descs([row_sum]), 0)
    assert names[0] and names[1] and not names[2] and not names[3]          # nothing stored elementwise
    assert names[8] == "ngh::red_rows_small_static_kernel<ngh::LP_b_0, false>" and names[9]
    chain = {"name": "jit_c", "type_name": "LP_c_0", "family": 4, "V": 4, "n_stat_slots": 0, "ops": [],
             "dtypes": [0, 0], "bcast": [0, 1], "rowshared": [0, 0], "staged": [-1, -1], "red_out": [],
             "stages": [dict(row_sum, type_name="LP_c_0_0"), dict(ew, type_name="LP_c_0_1", dtypes=[0, 0, 0])]}
    descs = hiplib.program_descs([ew, chain])
    names = hiplib.program_kernels(descs, 1)
    assert names[0] == "ngh::row_chain_static_kernel<0, 4, ngh::LP_c_0_0, ngh::LP_c_0_1>"
    assert names[3] == "ngh::row_chain_static_kernel<2, 8, ngh::LP_c_0_0, ngh::LP_c_0_1>" and not any(names[4:])
    with pytest.raises(hiplib.HipLibraryError, match="stage of chain"):
        hiplib.program_kernels(descs, 2)
    with pytest.raises(hiplib.HipLibraryError):
        hiplib.program_kernels(descs, 9)
    bad = hiplib.program_descs([dict(ew, V=3)])
    with pytest.raises(hiplib.HipLibraryError, match="malformed"):
        hiplib.program_kernels(bad, 0)


@pytest.mark.gpu
def test_a_code_bundle_that_does_not_fit_its_descriptions_is_refused(hip_runtime, tmp_path, monkeypatch):
    """ngh_programs_load_code checks what it is given before it publishes anything: the number
    of lowered names, names the code object does not hold."""
    import ctypes
    from ngraph_hip.runtime import hiplib
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    monkeypatch.setenv("NGH_JIT_COMPILER", "hiprtc")
    t, kernels = _dry_kernels(jit_cases.case_elementwise)
    try:
        path = jit.compile_programs(jit.uncovered_programs(kernels, "case")[:1])
    finally:
        t.close()
    dicts, lowered, code = hiplib.read_code_bundle(path)
    descs = hiplib.program_descs(dicts)
    lib, n = hip_runtime.lib, ctypes.c_int32()
    buf = ctypes.create_string_buffer(code, len(code))

    def load(names):
        return lib.ngh_programs_load_code(hip_runtime.ctx, ctypes.cast(buf, ctypes.c_void_p), len(code),
                                          ctypes.cast(descs, ctypes.c_void_p), len(descs), names.encode(), ctypes.byref(n))
    before = ctypes.c_int32()
    lib.ngh_programs_count(None, ctypes.byref(before))
    assert load(lowered + "\n") != 0 and b"lines" in lib.ngh_last_error()
    wrong = "\n".join(("_Z9not_there" if line else "") for line in lowered.split("\n")[:-1]) + "\n"
    assert load(wrong) != 0 and b"no kernel" in lib.ngh_last_error()
    missing = "\n" * hiplib.NGH_PROGRAM_KERNEL_SLOTS
    assert load(missing) != 0 and b"missing" in lib.ngh_last_error()
    after = ctypes.c_int32()
    lib.ngh_programs_count(None, ctypes.byref(after))
    assert after.value == before.value                      # nothing was added by the refused calls
    assert load(lowered) == 0                                # and the bundle as it was written loads


def test_without_hipcc_programs_are_compiled_in_process(tmp_path, monkeypatch):
    """A machine without hipcc: the same program becomes a code bundle made by hiprtc -- the
    descriptions of its programs, one lowered kernel name per slot the library asked for, and a
    code object."""
    import build_ext
    from ngraph_hip.runtime import hiplib

    def no_hipcc():
        raise RuntimeError("hipcc not found")
    from ngraph_hip.runtime import hiprtc
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    monkeypatch.delenv("NGH_JIT_COMPILER", raising=False)
    monkeypatch.setattr(build_ext, "find_hipcc", no_hipcc)
    assert jit.compiler() == "hiprtc"
    with monkeypatch.context() as m:             # (no libhiprtc either: hipcc is what is asked for)
        m.setattr(hiprtc, "available", lambda: False)
        assert jit.compiler() == "hipcc"
    for case, family in ((jit_cases.case_elementwise, 0), (jit_cases.case_softmax, 4),
                         (jit_cases.case_softmax_over_classes, 5)):
        t, kernels = _dry_kernels(case)
        try:
            programs = jit.uncovered_programs(kernels, "case")
            path = jit.compile_programs(programs[:1])
            assert path.endswith(hiplib.CODE_BUNDLE_SUFFIX) and path == jit.library_path_of(programs[:1])
            dicts, lowered, code = hiplib.read_code_bundle(path)
            assert len(dicts) == 1 and dicts[0]["family"] == family and dicts[0]["name"].startswith("jit_")
            names = lowered.split("\n")[:-1]
            assert len(names) == hiplib.NGH_PROGRAM_KERNEL_SLOTS
            wanted = hiplib.program_kernels(hiplib.program_descs(dicts), 0)
            assert [bool(n) for n in names] == [bool(w) for w in wanted] and any(names)
            assert all(n.startswith("_Z") for n in names if n)
            assert code[:4] == b"\x7fELF" and all(n.encode() in code for n in names if n)
            if family >= 4:
                assert len(dicts[0]["stages"]) == 3
        finally:
            t.close()


def test_missing_compiler_is_reported_as_such(tmp_path, monkeypatch):
    import build_ext

    def no_hipcc():
        raise RuntimeError("hipcc not found")
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    monkeypatch.setenv("NGH_JIT_COMPILER", "hipcc")          # (left to itself it would turn to hiprtc)
    monkeypatch.setattr(build_ext, "find_hipcc", no_hipcc)
    t, kernels = _dry_kernels(jit_cases.case_elementwise)
    try:
        with pytest.raises(RuntimeError, match="needs hipcc"):
            jit.compile_programs(jit.uncovered_programs(kernels, "case"))
    finally:
        t.close()


def test_default_mode_compiles_large_stages_in_the_background(monkeypatch):
    monkeypatch.delenv("NGH_JIT", raising=False)
    t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
    assert t.jit == "auto"
    t.close()
    for value, mode in (("1", True), ("0", False), ("auto", "auto")):
        monkeypatch.setenv("NGH_JIT", value)
        t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
        assert t.jit == mode and (t.jit is mode or mode == "auto")
        t.close()
    t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit=False)()
    assert t.jit is False
    t.close()
    with pytest.raises(ValueError):
        ngt.make_transformer_factory("hipgpu", dry_run=True, jit="sometimes")()


def test_background_programs_load_when_ready_and_only_for_large_stages(tmp_path, monkeypatch):
    """jit="auto": nothing is compiled for a small computation; for a large one the libraries are
    compiled by a worker thread and loaded by the kernel group once they exist; a second
    transformer finds them in the cache and loads them when its kernels are bound."""
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    results, inputs = jit_cases.case_elementwise()            # 512 x 1024 elements
    t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit="auto")()
    try:
        f = t.computation(results, *inputs)
        t.initialize()
        group = t.kernel_groups[f]
        group.bind()
        assert group._programs is None and not os.listdir(str(tmp_path))
    finally:
        t.close()
    for expect_thread in (True, False):
        t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit="auto", jit_auto_min_elements=1 << 18,
                                         jit_after_calls=2)()
        try:
            results, inputs = jit_cases.case_elementwise()
            f = t.computation(results, *inputs)
            t.initialize()
            group = t.kernel_groups[f]
            group.bind()
            assert (group._programs is not None) and not group._programs.started
            assert bool(group._programs._todo) == expect_thread
            group()                            # first run: nothing is compiled for it
            if expect_thread:
                assert not group._programs.started and not os.listdir(str(tmp_path))
                group()                        # second run: the compile jobs start
                assert group._programs.started
            assert group.wait_for_programs(timeout=300) is None
            assert group._programs is None
            libs = [n for n in os.listdir(str(tmp_path)) if n.endswith(".so") or n.endswith(".ngco")]
            assert len(libs) == 1 and t.runtime.program_libraries == [os.path.join(str(tmp_path), libs[0])]
        finally:
            t.close()


def test_by_default_compilation_starts_when_the_transformer_is_initialised(tmp_path, monkeypatch):
    """The reference compiles a computation's kernels at initialize() (float_ew2.py:1553-1653);
    the default mode hands the large stages to the compile workers at that point, before any run."""
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit="auto", jit_auto_min_elements=1 << 18)()
    try:
        results, inputs = jit_cases.case_elementwise()
        f = t.computation(results, *inputs)
        t.initialize()
        group = t.kernel_groups[f]
        assert group._bound and group._programs is not None and group._programs.started
        assert group.wait_for_programs(timeout=300) is None
        assert len([n for n in os.listdir(str(tmp_path)) if n.endswith(".so") or n.endswith(".ngco")]) == 1
    finally:
        t.close()


def test_background_compilation_without_a_compiler_stays_on_the_interpreter(tmp_path, monkeypatch):
    import build_ext

    def no_hipcc():
        raise RuntimeError("hipcc not found")
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    monkeypatch.setenv("NGH_JIT_COMPILER", "hipcc")          # (neither compiler: hiprtc is not asked)
    monkeypatch.setattr(build_ext, "find_hipcc", no_hipcc)
    t = ngt.make_transformer_factory("hipgpu", dry_run=True, jit="auto", jit_auto_min_elements=1 << 18)()
    try:
        results, inputs = jit_cases.case_elementwise()
        f = t.computation(results, *inputs)
        t.initialize()
        group = t.kernel_groups[f]
        group()                                              # runs (here: records) its launches
        error = group.wait_for_programs(timeout=60)
        assert error is not None and "needs hipcc" in error
        assert t.runtime.program_libraries == []
        group()
    finally:
        t.close()


def _run(backend, case, seed, **kwargs):
    t = ngt.make_transformer_factory(backend, **kwargs)()
    try:
        results, inputs = case()
        f = t.computation(results, *inputs)
        out = [np.array(r).copy() for r in f(*jit_cases.inputs_for(inputs, seed))]
        groups = getattr(t, "kernel_groups", None)
        names = [d for k in groups[f].kernels for ds in k.describe() for d in ds] if groups else []
        return out, names
    finally:
        t.close()


@pytest.mark.gpu
def test_auto_mode_swaps_compiled_kernels_in_without_changing_results(tmp_path, monkeypatch):
    """The default mode on the device: the first call runs on the interpreter while hipcc works
    (an empty cache, so this test does compile one program on the spot), later calls on the
    compiled kernel, and both give the same bits."""
    monkeypatch.setenv("NGH_PROGRAM_CACHE", str(tmp_path))
    t = ngt.make_transformer_factory("hipgpu", jit="auto", jit_auto_min_elements=1 << 18)()
    try:
        results, inputs = jit_cases.case_elementwise()
        f = t.computation(results, *inputs)
        vals = jit_cases.inputs_for(inputs, 3)
        group_names = lambda: [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
        first = [np.array(r).copy() for r in f(*vals)]
        before = group_names()
        assert t.kernel_groups[f].wait_for_programs(timeout=300) is None
        second = [np.array(r).copy() for r in f(*vals)]
        after = group_names()
        if default_kernel_choice():
            assert any("interp" in d for d in before) or any("special:jit_" in d for d in before), before
            assert all(d.startswith("special:jit_") for d in after), after
        for a, b in zip(first, second):
            np.testing.assert_array_equal(a, b)
    finally:
        t.close()


COLUMN_SOFTMAX_CASES = (jit_cases.case_softmax_over_classes, jit_cases.case_softmax_over_few_classes,
                        jit_cases.case_softmax_over_ten_classes_of_many_samples, jit_cases.case_column_statistics_chain)


@pytest.mark.gpu
@pytest.mark.parametrize("case", jit_cases.FP32_CASES, ids=lambda c: c.__name__)
def test_compiled_programs_agree_with_the_interpreter(case):
    import oracle.cpu_transformer  # noqa: F401
    want, _ = _run("cpu", case, 5)
    interp, names_interp = _run("hipgpu", case, 5, jit=False)
    compiled, names = _run("hipgpu", case, 5, jit=True)
    # Same bits as the interpreter -- except where the compiled program runs 4 elements per lane
    # over rows that are not whole aligned vectors (the interpreter takes those one element per
    # lane), or several stages as one row-chain kernel: a reduction then adds up in another order.
    # (and a compiled reduction across the contiguous axis splits the reduced axis into fewer,
    # longer segments than the interpreted one: the softmax over classes when its stages run apart)
    ragged = any("/ragged" in n or "chain-of-" in n for n in names) or case in COLUMN_SOFTMAX_CASES
    for a, b, w in zip(interp, compiled, want):
        half = np.asarray(b).dtype == np.float16
        if ragged and half:
            # (a sum added up in another order can put a result on the neighbouring fp16 value)
            np.testing.assert_allclose(a, b, rtol=1e-3, atol=1e-6)
            assert (np.asarray(a) != np.asarray(b)).mean() < 1e-3
        elif ragged:
            np.testing.assert_allclose(a, b, rtol=2e-6, atol=1e-6)
        else:
            np.testing.assert_array_equal(a, b)
        if case is jit_cases.case_dropout:
            # the oracle draws from NumPy's generator: only the distribution is comparable
            assert abs(np.count_nonzero(compiled[0]) / compiled[0].size - 0.75) < 0.01
        else:
            np.testing.assert_allclose(b, w, rtol=1e-3 if half else 1e-5, atol=1e-5)
    if default_kernel_choice():
        # every stage large enough to be worth a compiled kernel has one now
        assert not any("interp" in n for n in names if "tail" not in n), names
        if case in (jit_cases.case_ragged, jit_cases.case_ragged_long_rows, jit_cases.case_ragged_many_rows,
                    jit_cases.case_misaligned_slices):
            assert any(n.endswith("/ragged") for n in names), names
        if case in (jit_cases.case_softmax, jit_cases.case_softmax_ragged_rows, jit_cases.case_short_rows,
                    jit_cases.case_softmax_of_half_rows,
                    jit_cases.case_softmax_long_rows, jit_cases.case_softmax_over_windows,
                    jit_cases.case_softmax_forward_and_backward,
                    jit_cases.case_row_chain_with_stored_intermediate, jit_cases.case_row_statistics_chain):
            assert any("/chain-of-" in n for n in names), names
        if case in (jit_cases.case_softmax_over_classes, jit_cases.case_softmax_over_few_classes,
                    jit_cases.case_softmax_over_ten_classes_of_many_samples, jit_cases.case_column_statistics_chain):
            assert any("/column-chain-of-3" in n for n in names), names
        if case is jit_cases.case_row_statistics_chain:
            # (the other way to the statistics is what ran before the chain was there)
            assert any("moments" in n for n in names_interp), names_interp
        if case is jit_cases.case_transposed_operands_large:
            assert any(n.endswith("/tiles64") for n in names), names


@pytest.mark.gpu
def test_programs_of_either_compiler_agree_with_the_interpreter():
    """The same cases with each compiler named explicitly, one child process per compiler (a
    program, once loaded, serves the whole process, whichever compiler made it): hiprtc -- kernels
    compiled inside the process (here: found as code bundles in the cache, where the CPU suite
    left them), loaded with hipModuleLoadData and launched with hipModuleLaunchKernel -- and
    hipcc -- shared objects with host launchers."""
    import json
    import subprocess
    import sys
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rtc_child.py")
    for compiler in ("hiprtc", "hipcc"):
        proc = subprocess.run([sys.executable, child, compiler], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                              timeout=900)
        assert proc.returncode == 0, proc.stderr.decode()[-2000:]
        report = json.loads(proc.stdout.decode().strip().splitlines()[-1])
        assert report["failures"] == [] and report["compiler"] == compiler, report
        if not default_kernel_choice():
            continue
        assert report["cases"] >= 26 and report["loaded"] >= 20 and report["compiled_kernels"] >= 40, report
        mine, other = ("code_bundles_loaded", "shared_objects_loaded") if compiler == "hiprtc" else \
            ("shared_objects_loaded", "code_bundles_loaded")
        assert report[mine] >= 20 and report[other] == 0, report


@pytest.mark.gpu
@pytest.mark.parametrize("views", [False, True], ids=["plain", "views"])
@pytest.mark.parametrize("seed", jit_cases.RANDOM_SEEDS)
def test_random_graphs_compiled_agree_with_the_interpreter(seed, views):
    def run(**kwargs):
        t = ngt.make_transformer_factory("hipgpu", **kwargs)()
        try:
            results, inputs, values = jit_cases.random_case(seed, views)
            f = t.computation(results, *inputs)
            out = [np.array(r).copy() for r in f(*values)]
            return out, [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
        finally:
            t.close()
    (interp, _), (compiled, names) = run(jit=False), run(jit=True, jit_min_elements=1)
    ragged = any("/ragged" in n or "chain-of-" in n for n in names)       # (see the test above)
    for a, b in zip(interp, compiled):
        if ragged:
            np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-5)
        else:
            np.testing.assert_array_equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("resident", [False, True], ids=["host-policy", "device-policy"])
def test_compiled_flex_program_agrees_with_the_interpreter(resident):
    """A flex kernel compiled at run time carries statistics slots like the built-in ones: in
    device-resident mode it takes the one-launch path with deferred statistics."""
    def run(use_jit):
        t = ngt.make_transformer_factory("flexhip", resident=resident, jit=use_jit)()
        try:
            results, inputs = jit_cases.flex_case()
            f = t.computation(results, *inputs)
            vals = jit_cases.inputs_for(inputs, 9)
            outs = [np.array(f(vals[0] * g, vals[1], vals[2])).copy() for g in (1.0, 4.0, 30.0, 0.1, 1.0)]
            names = [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
            return outs, names
        finally:
            t.close()
    a, _ = run(False)
    b, names = run(True)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    if default_kernel_choice():
        assert any(n.startswith("special:") for n in names), names


@pytest.mark.gpu
def test_loading_a_program_library_twice_adds_nothing():
    from ngraph_hip.runtime import HipRuntime
    t, kernels = _dry_kernels(jit_cases.case_ragged_long_rows)
    try:
        # (earlier tests of this process may have loaded these very programs)
        built_in = hiplib.programs_count()[0]
        programs = [p for p in jit.uncovered_programs(kernels, "case", include_covered=True)
                    if not 0 <= p[-1] < built_in]
        assert len(programs) == 3
        paths = [jit.compile_programs([p]) for p in programs]
        path = paths[0]
    finally:
        t.close()
    rt = HipRuntime(0)
    try:
        for p in paths:
            rt.programs_load(p)
        built_in, loaded = hiplib.programs_count()
        assert loaded >= 2
        assert rt.programs_load(path) == 0
        assert hiplib.programs_count() == (built_in, loaded)
        with pytest.raises(hiplib.HipLibraryError):
            rt.programs_load(os.path.join(os.path.dirname(path), "no_such_library.so"))
        # a shared object that is no program library
        with pytest.raises(hiplib.HipLibraryError, match="ngh_program_library"):
            rt.programs_load(hiplib.library_path())
    finally:
        rt.close()


# ---------------------------------------------------------------------------------- row chains
def _softmax_spec(px, pm, ps, py, R, rows, row_stride=None, x_dtype=hiplib.NGH_F32, only=None):
    """max / sum of exponentials / normalise over the rows of an [rows, R] tensor as three stages
    (only: just that one of them)."""
    stride = R if row_stride is None else row_stride
    sb = hiplib.FusedSpecBuilder([R, rows])
    tx, ty = sb.tensor(px, [1, stride], x_dtype), sb.tensor(py, [1, stride])
    tm, ts = sb.tensor(pm, [0, 1]), sb.tensor(ps, [0, 1])
    if only in (None, 0):
        sb.reduce("max", sb.load(tx), tm)
        sb.end_stage()
    if only in (None, 1):
        sb.reduce("sum", sb.unary("exp", sb.binary("sub", sb.load(tx), sb.load(tm))), ts)
        sb.end_stage()
    if only in (None, 2):
        e = sb.unary("exp", sb.binary("sub", sb.load(tx), sb.load(tm)))
        sb.store(ty, sb.binary("div", e, sb.load(ts)))
    return sb.build()


def test_which_specs_are_row_chains():
    """ngh_plan_chain without a device: rows of 8 to 8192 fp32 (or flex16 / fp16) elements with unit
    stride, at least one reduction stage, more than one stage."""
    if not default_kernel_choice():
        pytest.skip("a kernel-choice knob of the library is set")
    ok = lambda spec: hiplib.plan_chain(spec)["eligible"]
    assert ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300))
    assert hiplib.plan_chain(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300))["lanes_per_row"] == 64
    assert hiplib.plan_chain(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 100, 300))["lanes_per_row"] == 32
    assert hiplib.plan_chain(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 5000, 300))["lanes_per_row"] == 256
    assert ok(_softmax_spec((1 << 30) + 4, 2 << 30, 3 << 30, (4 << 30) + 4, 1000, 300, row_stride=1003))      # any 4-byte-aligned start
    assert not ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 7, 300))
    assert not ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 8193, 300))
    # 16-bit operands: every chunk of four on a 4-byte boundary (an aligned start, rows an even
    # number of elements apart); other integer storage stays out
    assert ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1000, 300, x_dtype=hiplib.NGH_FLEX16))
    assert ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300, row_stride=1002, x_dtype=hiplib.NGH_F16))
    assert not ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300, x_dtype=hiplib.NGH_FLEX16))
    assert not ok(_softmax_spec((1 << 30) + 2, 2 << 30, 3 << 30, 4 << 30, 1000, 300, x_dtype=hiplib.NGH_FLEX16))
    assert not ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1000, 300, x_dtype=hiplib.NGH_I16))
    # two operand slots over the same memory, one of them written: the stages must see each
    # other's writes, which the chain's registers would hide
    assert not ok(_softmax_spec(1 << 30, 2 << 30, 3 << 30, (1 << 30) + 4000, 1001, 300))
    assert ok(_aliased_chain_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300))
    assert not ok(_aliased_chain_spec(1 << 30, 2 << 30, 3 << 30, 1 << 30, 1001, 300))
    # rows that are strided in memory
    sb = hiplib.FusedSpecBuilder([64, 300])
    tx, tm, ty = sb.tensor(4096, [300, 1]), sb.tensor(8192, [0, 1]), sb.tensor(16384, [300, 1])
    sb.reduce("max", sb.load(tx), tm)
    sb.end_stage()
    sb.store(ty, sb.binary("sub", sb.load(tx), sb.load(tm)))
    assert not ok(sb.build())
    # one stage, and stages without a reduction
    sb = hiplib.FusedSpecBuilder([64, 300])
    sb.reduce("max", sb.load(sb.tensor(4096, [1, 64])), sb.tensor(8192, [0, 1]))
    assert not ok(sb.build())
    sb = hiplib.FusedSpecBuilder([64, 300])
    tx, ty, tz = sb.tensor(4096, [1, 64]), sb.tensor(16384, [1, 64]), sb.tensor(65536, [1, 64])
    sb.store(ty, sb.unary("exp", sb.load(tx)))
    sb.end_stage()
    sb.store(tz, sb.unary("tanh", sb.load(tx)))
    assert not ok(sb.build())


def _fenced_chain_spec(px, pi, pt, py, pn, R, rows):
    sb = hiplib.FusedSpecBuilder([R, rows])
    tx, ti = sb.tensor(px, [1, R]), sb.tensor(pi, [0, 1], hiplib.NGH_I32)
    tt, ty, tn = sb.tensor(pt, [1, R]), sb.tensor(py, [1, R]), sb.tensor(pn, [0, 1])
    sb.reduce("argmax", sb.load(tx), ti)
    sb.end_stage()
    # t = x * 2 + position of the row's maximum; n = sum(t * t)
    t = sb.binary("add", sb.binary("mul", sb.load(tx), sb.constant(2.0)), sb.load(ti))
    sb.store(tt, t)
    sb.reduce("sum", sb.binary("mul", t, t), tn)
    sb.end_stage()
    # y = t / sqrt(n), t read back from memory
    sb.store(ty, sb.binary("div", sb.load(tt), sb.unary("sqrt", sb.load(tn))))
    return sb.build()


def _aliased_chain_spec(px, pm, ps, pz, R, rows):
    """m = max(x); z = x - m; s = sum(exp(x)) with x read through its own slot in every stage.
    With z at x's address the third stage must see x - m."""
    sb = hiplib.FusedSpecBuilder([R, rows])
    tx, tz = sb.tensor(px, [1, R]), sb.tensor(pz, [1, R])
    tm, ts = sb.tensor(pm, [0, 1]), sb.tensor(ps, [0, 1])
    sb.reduce("max", sb.load(tx), tm)
    sb.end_stage()
    sb.store(tz, sb.binary("sub", sb.load(tx), sb.load(tm)))
    sb.end_stage()
    sb.reduce("sum", sb.unary("exp", sb.load(tx)), ts)
    return sb.build()


def test_row_chain_specs_compile_for_gfx950():
    """(also leaves their program libraries in the cache for the device tests below)"""
    for spec in (_softmax_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 1001, 300),
                 _fenced_chain_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 5 << 30, 777, 3000),
                 _aliased_chain_spec(1 << 30, 2 << 30, 3 << 30, 4 << 30, 500, 2000)):
        programs = jit.uncovered_programs([_SpecHolder(spec)], "chain", min_elements=1, include_covered=True)
        if default_kernel_choice():
            assert len(programs) == 1 and programs[0][8] == 4
        assert not programs or os.path.exists(jit.compile_programs(programs))


class _SpecHolder(object):
    def __init__(self, spec):
        self.specs = [spec]


@pytest.mark.gpu
@pytest.mark.parametrize("rows,R,stride", [(300, 1001, None), (5000, 100, None), (2000, 16, None), (64, 8192, None),
                                           (70, 4099, None), (301, 1000, 1003), (1, 9, None)])
def test_row_chain_through_the_c_abi(hip_runtime, rows, R, stride, monkeypatch):
    """A three-stage softmax spec: launched as one chain kernel it gives what its stages give when
    launched one by one, and what NumPy gives."""
    rt = hip_runtime
    stride = R if stride is None else stride
    rs = np.random.RandomState(rows + R)
    x = rs.normal(0, 3, (rows, stride)).astype(np.float32)
    x_d = rt.array(x)
    outs = {}
    for chained in (True, False):
        m_d, s_d, y_d = rt.empty((rows,)), rt.empty((rows,)), rt.empty((rows, stride))
        rt.memset32(y_d.ptr, 0x7fc00000, rows * stride)
        spec = _softmax_spec(x_d.ptr, m_d.ptr, s_d.ptr, y_d.ptr, R, rows, row_stride=stride)
        jit.ensure_programs(rt, [_SpecHolder(spec)], "softmax_chain", min_elements=1)
        if chained:
            if default_kernel_choice():
                assert "/chain-of-3" in rt.describe_fused(spec, 0)
            rt.launch_fused(spec)
        else:
            # the same stages, each a spec of its own
            for stage in range(3):
                one = _softmax_spec(x_d.ptr, m_d.ptr, s_d.ptr, y_d.ptr, R, rows, row_stride=stride, only=stage)
                assert "chain" not in rt.describe_fused(one, 0)
                rt.launch_fused(one)
        outs[chained] = (m_d.get(), s_d.get(), y_d.get())
        for d in (m_d, s_d, y_d):
            d.free()
    x_d.free()
    x64 = x[:, :R].astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    for m, s, y in outs.values():
        np.testing.assert_array_equal(m, x[:, :R].max(axis=1))
        np.testing.assert_allclose(s, e.sum(axis=1), rtol=1e-5)
        np.testing.assert_allclose(y[:, :R], e / e.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-6)
        assert np.isnan(y[:, R:]).all()                  # the gap between rows is not written
    np.testing.assert_allclose(outs[True][2][:, :R], outs[False][2][:, :R], rtol=2e-6, atol=1e-7)


@pytest.mark.gpu
def test_row_chain_with_results_that_go_through_memory(hip_runtime):
    """What the stages of a chain cannot hand on in registers goes through memory behind a fence:
    the position of the maximum (kept as int32) read back by the next stage, and a tensor that
    one stage stores and the next loads."""
    rt = hip_runtime
    rows, R = 3000, 777
    rs = np.random.RandomState(5)
    x = rs.normal(0, 1, (rows, R)).astype(np.float32)
    x_d, i_d, t_d, y_d, n_d = rt.array(x), rt.empty((rows,), hiplib.NGH_I32), rt.empty((rows, R)), rt.empty((rows, R)), \
        rt.empty((rows,))
    spec = _fenced_chain_spec(x_d.ptr, i_d.ptr, t_d.ptr, y_d.ptr, n_d.ptr, R, rows)
    assert hiplib.plan_chain(spec)["eligible"] or not default_kernel_choice()
    jit.ensure_programs(rt, [_SpecHolder(spec)], "fenced_chain", min_elements=1)
    if default_kernel_choice():
        assert "/chain-of-3" in rt.describe_fused(spec, 0)
    rt.launch_fused(spec)
    pos = x.argmax(axis=1)
    np.testing.assert_array_equal(i_d.get(), pos)
    t_want = x.astype(np.float64) * 2.0 + pos[:, None]
    n_want = (t_want * t_want).sum(axis=1)
    np.testing.assert_allclose(t_d.get(), t_want, rtol=1e-6)
    np.testing.assert_allclose(n_d.get(), n_want, rtol=1e-5)
    np.testing.assert_allclose(y_d.get(), t_want / np.sqrt(n_want)[:, None], rtol=1e-5, atol=1e-7)
    for d in (x_d, i_d, t_d, y_d, n_d):
        d.free()


@pytest.mark.gpu
@pytest.mark.parametrize("R", [500, 5000])
def test_operand_slots_over_the_same_memory_never_run_as_a_chain(hip_runtime, R):
    """A spec whose second stage writes, through a slot of its own, the memory its first and
    third stages read: with the chain's program loaded the unaliased spec runs as one kernel,
    the aliased one stage by stage, and the third stage sees what the second wrote."""
    rt = hip_runtime
    rows = 2000
    x = np.random.RandomState(R).normal(0, 2, (rows, R)).astype(np.float32)
    x_d, z_d, m_d, s_d = rt.array(x), rt.empty((rows, R)), rt.empty((rows,)), rt.empty((rows,))
    apart = _aliased_chain_spec(x_d.ptr, m_d.ptr, s_d.ptr, z_d.ptr, R, rows)
    jit.ensure_programs(rt, [_SpecHolder(apart)], "aliased_chain", min_elements=1)
    if default_kernel_choice():
        assert "/chain-of-3" in rt.describe_fused(apart, 0)
    rt.launch_fused(apart)
    m = x.max(axis=1)
    np.testing.assert_array_equal(z_d.get(), x - m[:, None])
    np.testing.assert_allclose(s_d.get(), np.exp(x.astype(np.float64)).sum(axis=1), rtol=1e-5)
    aliased = _aliased_chain_spec(x_d.ptr, m_d.ptr, s_d.ptr, x_d.ptr, R, rows)
    assert "chain" not in rt.describe_fused(aliased, 0)
    rt.launch_fused(aliased)
    shifted = x - m[:, None]
    np.testing.assert_array_equal(x_d.get(), shifted)
    np.testing.assert_allclose(s_d.get(), np.exp(shifted.astype(np.float64)).sum(axis=1), rtol=1e-5)
    for d in (x_d, z_d, m_d, s_d):
        d.free()


@pytest.mark.gpu
def test_chained_kernels_run_by_themselves_until_the_chain_is_compiled():
    """Without a compiled chain (run-time compilation off, no such chain built in) the merged
    kernels keep running one by one, with the programs they match by themselves; with
    compilation on the same graph is one launch.  Same results either way."""
    def run(**kwargs):
        t = ngt.make_transformer_factory("hipgpu", **kwargs)()
        try:
            C, N = ng.make_axis(700, name="C"), ng.make_axis(3000, name="N")
            x = ng.placeholder([N, C])
            e = ng.exp((x - ng.max(x, out_axes=[N])) * 0.5)
            f = t.computation(e / ng.sum(e, out_axes=[N]), x)
            xv = np.random.RandomState(2).normal(0, 2, (3000, 700)).astype(np.float32)
            out = np.array(f(xv)).copy()
            names = [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
            return out, names, xv
        finally:
            t.close()
    alone, names_alone, xv = run(jit=False)
    chained, names_chained, _ = run(jit=True, jit_min_elements=1)
    if default_kernel_choice():
        assert not any("/chain-of-" in n for n in names_alone), names_alone
        assert "special:max_along_k0" in names_alone[0], names_alone        # the built-in row maximum
        assert len(names_chained) == 3 and all("/chain-of-3" in n for n in names_chained), names_chained
    e = np.exp((xv.astype(np.float64) - xv.max(axis=1, keepdims=True)) * 0.5)
    want = e / e.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(alone, want, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(chained, want, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_row_statistics_and_their_consumer_merge_into_a_chain():
    """mean / variance of rows (one MomentsOp in the graph) and the kernel that normalises with
    them: one chain -- sum, sum of squared deviations, normalise; with the statistics returned
    as well, a stage in between that writes them out, one value per row.  Without a compiled
    chain: the one-pass moments kernel and the normalise kernel as before."""
    def run(with_stats, **kwargs):
        t = ngt.make_transformer_factory("hipgpu", **kwargs)()
        try:
            N, C = ng.make_axis(2500, name="N"), ng.make_axis(777, name="C")
            x, g, b = ng.placeholder([N, C]), ng.placeholder([C]), ng.placeholder([C])
            mean, var = ng.mean(x, out_axes=[N]), ng.variance(x, out_axes=[N])
            y = g * ((x - mean) * ng.reciprocal(ng.sqrt(var + 1e-5))) + b
            f = t.computation([y, mean, var] if with_stats else [y], x, g, b)
            rs = np.random.RandomState(8)
            xv = rs.normal(0.5, 2.0, (2500, 777)).astype(np.float32)
            gv, bv = rs.uniform(0.5, 1.5, 777).astype(np.float32), rs.uniform(-1, 1, 777).astype(np.float32)
            out = [np.array(r).copy() for r in f(xv, gv, bv)]
            names = [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
            return out, names, (xv, gv, bv)
        finally:
            t.close()
    # (first without compilation: a program, once loaded, serves every transformer of the process)
    alone, names_alone, _ = run(False, jit=False)
    chained, names_chained, (xv, gv, bv) = run(False, jit=True, jit_min_elements=1)
    with_stats, names_stats, _ = run(True, jit=True, jit_min_elements=1)
    if default_kernel_choice():
        assert all("/chain-of-3" in n for n in names_chained) and len(names_chained) == 3, names_chained
        # (unless an earlier test of this process has loaded this very chain already)
        assert names_alone[0] == "moments_f32" or all("/chain-of-3" in n for n in names_alone), names_alone
        assert all("/chain-of-4" in n for n in names_stats) and len(names_stats) == 4, names_stats
    x64 = xv.astype(np.float64)
    m, v = x64.mean(axis=1, keepdims=True), x64.var(axis=1, keepdims=True)
    want = gv * ((x64 - m) / np.sqrt(v + 1e-5)) + bv
    for got in (chained[0], alone[0], with_stats[0]):
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(with_stats[1], m[:, 0], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(with_stats[2], v[:, 0], rtol=1e-5, atol=1e-6)


def _row_store_spec(px, ps, pm, R, rows, varying=False):
    """sum of rows, then a stage that stores one value per row (the mean)."""
    sb = hiplib.FusedSpecBuilder([R, rows])
    tx, ts, tm = sb.tensor(px, [1, R]), sb.tensor(ps, [0, 1]), sb.tensor(pm, [0, 1])
    sb.reduce("sum", sb.load(tx), ts)
    sb.end_stage()
    mean = sb.binary("div", sb.load(ts), sb.constant(float(R)))
    sb.store(tm, sb.binary("add", mean, sb.load(tx)) if varying else mean)
    return sb


def test_one_value_per_row_may_be_stored_only_if_it_is_the_same_along_the_row():
    from ngraph_hip.runtime.hiplib import DryRunRuntime
    rt = DryRunRuntime()
    rt.validate_fused(_row_store_spec(4096, 8192, 12288, 100, 50).build())
    with pytest.raises(hiplib.HipLibraryError, match="broadcast along axis 0"):
        rt.validate_fused(_row_store_spec(4096, 8192, 12288, 100, 50, varying=True).build())


@pytest.mark.gpu
def test_a_spec_that_stores_one_value_per_row_runs_as_a_chain_or_not_at_all(hip_runtime):
    rt = hip_runtime
    rows, R = 1500, 333
    x = np.random.RandomState(3).normal(1.0, 2.0, (rows, R)).astype(np.float32)
    x_d, s_d, m_d = rt.array(x), rt.empty((rows,)), rt.empty((rows,))
    spec = _row_store_spec(x_d.ptr, s_d.ptr, m_d.ptr, R, rows).build()
    if hiplib.plan_chain(spec)["special"] < 0:
        with pytest.raises(hiplib.HipLibraryError, match="row chain"):
            rt.launch_fused(spec)
    if default_kernel_choice():
        jit.ensure_programs(rt, [_SpecHolder(spec)], "row_store", min_elements=1)
        assert "/chain-of-2" in rt.describe_fused(spec, 0)
        rt.launch_fused(spec)
        np.testing.assert_allclose(m_d.get(), x.astype(np.float64).mean(axis=1), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(s_d.get(), x.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-4)
    for d in (x_d, s_d, m_d):
        d.free()


@pytest.mark.gpu
def test_normalisations_over_short_rows_run_as_built_in_chains():
    """Batch normalisation as the neon front writes it, layer normalisation and (log-)softmax over
    rows of up to 8192 elements: one launch each from chains built into the library, without
    run-time compilation."""
    from ngraph_hip.frontends import neon
    rs = np.random.RandomState(4)
    t = ngt.make_transformer_factory("hipgpu", jit=False)()
    try:
        C, H, W, N = (ng.make_axis(n, name=k) for k, n in zip("CHWN", (48, 9, 9, 32)))
        x = ng.placeholder([C, H, W, N])
        gv, bv = rs.uniform(0.5, 1.5, 48).astype(np.float32), rs.uniform(-1, 1, 48).astype(np.float32)
        gamma, beta = ng.variable([C], initial_value=gv), ng.variable([C], initial_value=bv)
        y, mean, var = neon.batch_norm_train(x, gamma, beta, out_axes=[C])
        bn = t.computation([y, mean, var], x)
        R, K = ng.make_axis(700, name="R"), ng.make_axis(1500, name="K")
        w = ng.placeholder([R, K])
        mu, vv = ng.mean(w, out_axes=[R]), ng.variance(w, out_axes=[R])
        ln = t.computation((w - mu) * ng.reciprocal(ng.sqrt(vv + 1e-5)), w)
        sm = t.computation(ng.softmax(w, normalization_axes=ng.make_axes([K])), w)
        xv = rs.normal(0.5, 2.0, (48, 9, 9, 32)).astype(np.float32)
        wv = rs.normal(0.0, 3.0, (700, 1500)).astype(np.float32)
        y_, mean_, var_ = [np.array(a) for a in bn(xv)]
        ln_, sm_ = np.array(ln(wv)), np.array(sm(wv))
        if default_kernel_choice():
            for f, name, stages in ((bn, "batchnorm_short_rows_k0", 4), (ln, "layer_norm_rows_k0", 3), (sm, "softmax_rows_k0", 3)):
                names = [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
                assert names == ["special:%s/chain-of-%d" % (name, stages)] * stages, names
    finally:
        t.close()
    x64 = xv.astype(np.float64).reshape(48, -1)
    m, v = x64.mean(axis=1), x64.var(axis=1)
    np.testing.assert_allclose(mean_, m, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(var_, v, rtol=1e-5, atol=1e-6)
    want = gv[:, None] * (x64 - m[:, None]) / np.sqrt(v[:, None] + 1e-5) + bv[:, None]
    np.testing.assert_allclose(y_.reshape(48, -1), want, rtol=1e-5, atol=2e-6)
    w64 = wv.astype(np.float64)
    np.testing.assert_allclose(ln_, (w64 - w64.mean(axis=1, keepdims=True)) / np.sqrt(w64.var(axis=1, keepdims=True) + 1e-5),
                               rtol=1e-5, atol=2e-6)
    e = np.exp(w64 - w64.max(axis=1, keepdims=True))
    np.testing.assert_allclose(sm_, e / e.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_compiled_flex_fill_truncates_like_the_interpreter():
    """A fill of a flex16 tensor stores int(value / scale) cut toward zero (the reference's
    FlexFillKernel, tensor_ops.py:690-707): compiled at run time and interpreted give the same
    mantissas and exponent, for values that round differently from how they are cut."""
    def run(use_jit):
        t = ngt.make_transformer_factory("flexhip", jit=use_jit, jit_min_elements=1)()
        try:
            P = ng.make_axis(1 << 16, name="P")
            v = ng.variable([P], initial_value=0)
            out, names = [], []
            fills = [t.computation(ng.sequential([ng.fill(v, value), v * 1.0])) for value in (1.2, -1.7, 0.99999, 3.0)]
            for f in fills:
                f()
                view = t.get_op_tensor_view(v)
                out.append((view._read_raw().copy(), view.flex_entry.dec))
                names += [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
            return out, names
        finally:
            t.close()
    a, names_interp = run(False)
    b, names = run(True)
    for (ma, da), (mb, db) in zip(a, b):
        assert da == db
        np.testing.assert_array_equal(ma, mb)
    # cut toward zero: 1.2 at the exponent of the variable's first use
    first, dec = b[0]
    assert (first == int(np.trunc(np.float32(1.2) * np.float32(2.0 ** dec)))).all()
    if default_kernel_choice():
        assert any(n.startswith("special:jit_") for n in names), names
        assert not any(n.startswith("special:") for n in names_interp), names_interp


@pytest.mark.gpu
def test_flex_computation_picks_up_programs_compiled_in_the_background():
    """jit="auto" with the flex transformer: once every exponent is initialised the kernel group
    makes one library call per kernel and nothing else; it still has to load what the compile
    workers finish, or the computation would stay on the interpreter for good."""
    import time
    t = ngt.make_transformer_factory("flexhip", jit="auto", jit_auto_min_elements=1, jit_min_elements=1)()
    try:
        P = ng.make_axis(1 << 16, name="P")
        x, w = ng.placeholder([P]), ng.placeholder([P])
        f = t.computation(ng.tanh(x * w + 0.25) * 1.5 - x, x, w)      # (a program no other test compiles)
        vals = jit_cases.inputs_for([x, w], 21)
        f(*vals)
        group = t.kernel_groups[f]
        names = []
        for _ in range(400):
            out = np.array(f(*vals)).copy()
            names = [d for k in group.kernels for ds in k.describe() for d in ds]
            if default_kernel_choice() and any(n.startswith("special:jit_") for n in names):
                break
            time.sleep(0.05)
        want = np.tanh(vals[0].astype(np.float64) * vals[1] + 0.25) * 1.5 - vals[0]
        atol, rtol = t.get_default_tolerance(want)
        np.testing.assert_allclose(out, want, rtol=rtol, atol=atol)
        if default_kernel_choice():
            assert any(n.startswith("special:jit_") for n in names), names
    finally:
        t.close()
