"""Run by tests/test_jit.py::test_programs_of_either_compiler_agree_with_the_interpreter in a
process of its own, with the compiler's name as its argument: every case of jit_cases with its
programs compiled by that compiler (hiprtc: inside the process, launched through the module
API; hipcc: shared objects with host launchers), against the interpreter and the oracle.  (A
process of its own because a program, once loaded, serves the whole process: the other
compiler's libraries would be taken for known and skipped.)  Prints one JSON line."""
import json
import os
import sys

os.environ["NGH_JIT_COMPILER"] = sys.argv[1] if len(sys.argv) > 1 else "hiprtc"
os.environ.pop("NGH_JIT", None)
HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [HERE, os.path.dirname(HERE), os.path.join(os.path.dirname(HERE), "ngraph-python_amd")]

import numpy as np  # noqa: E402

import ngraph_hip.transformers as ngt  # noqa: E402
from ngraph_hip.runtime import hiplib  # noqa: E402
import jit_cases  # noqa: E402
from conftest import default_kernel_choice  # noqa: E402
import oracle.cpu_transformer  # noqa: E402,F401


LOADED = []           # the libraries the runtimes of this process were given


def run(backend, case, seed, **kwargs):
    t = ngt.make_transformer_factory(backend, **kwargs)()
    try:
        results, inputs = case()
        f = t.computation(results, *inputs)
        out = [np.array(r).copy() for r in f(*jit_cases.inputs_for(inputs, seed))]
        groups = getattr(t, "kernel_groups", None)
        names = [d for k in groups[f].kernels for ds in k.describe() for d in ds] if groups else []
        return out, names
    finally:
        LOADED.extend(getattr(getattr(t, "runtime", None), "program_libraries", []))
        t.close()


def main():
    failures, compiled_names = [], 0
    for case in jit_cases.FP32_CASES:
        try:
            want, _ = run("cpu", case, 5)
            interp, _ = run("hipgpu", case, 5, jit=False)
            compiled, names = run("hipgpu", case, 5, jit=True)
            reordered = any("/ragged" in n or "chain-of-" in n for n in names) or "over_classes" in case.__name__ \
                or "over_few_classes" in case.__name__ or "ten_classes" in case.__name__ or "column_statistics" in case.__name__
            for a, b, w in zip(interp, compiled, want):
                half = np.asarray(b).dtype == np.float16       # (an fp16 result may land on the neighbouring value)
                if reordered:
                    np.testing.assert_allclose(a, b, rtol=1e-3 if half else 2e-6, atol=1e-6)
                else:
                    np.testing.assert_array_equal(a, b)
                if case is not jit_cases.case_dropout:
                    np.testing.assert_allclose(b, w, rtol=1e-3 if half else 1e-5, atol=1e-5)
            if default_kernel_choice() and any("interp" in n for n in names if "tail" not in n):
                raise AssertionError("still interpreted: %s" % names)
            compiled_names += sum(1 for n in names if n.startswith("special:jit_"))
        except Exception as e:
            failures.append("%s: %s" % (case.__name__, str(e)[:300]))
    # a flex kernel: statistics slots, the deferred-statistics variants
    def run_flex(resident, use_jit):
        t = ngt.make_transformer_factory("flexhip", resident=resident, jit=use_jit)()
        try:
            results, inputs = jit_cases.flex_case()
            f = t.computation(results, *inputs)
            vals = jit_cases.inputs_for(inputs, 9)
            outs = [np.array(f(vals[0] * g, vals[1], vals[2])).copy() for g in (1.0, 4.0, 30.0, 0.1, 1.0)]
            return outs, [d for k in t.kernel_groups[f].kernels for ds in k.describe() for d in ds]
        finally:
            LOADED.extend(t.runtime.program_libraries)
            t.close()

    for resident in (False, True):
        try:
            a, _ = run_flex(resident, False)
            b, names = run_flex(resident, True)
            for x, y in zip(a, b):
                np.testing.assert_array_equal(x, y)
            compiled_names += sum(1 for n in names if n.startswith("special:jit_"))
        except Exception as e:
            failures.append("flex_case resident=%s: %s" % (resident, str(e)[:300]))
    lib = hiplib.load_library()
    import ctypes
    built_in, loaded = ctypes.c_int32(), ctypes.c_int32()
    lib.ngh_programs_count(ctypes.byref(built_in), ctypes.byref(loaded))
    print(json.dumps({"cases": len(jit_cases.FP32_CASES) + 2, "failures": failures, "loaded": loaded.value,
                      "compiled_kernels": compiled_names, "compiler": os.environ["NGH_JIT_COMPILER"],
                      "code_bundles_loaded": len(set(p for p in LOADED if p.endswith(hiplib.CODE_BUNDLE_SUFFIX))),
                      "shared_objects_loaded": len(set(p for p in LOADED if p.endswith(".so")))}))


if __name__ == "__main__":
    main()
