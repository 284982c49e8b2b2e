"""bench.py and __graft_entry__ behaviour that needs no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert p.returncode != 0
    assert "one GPU" in p.stderr
    assert not p.stdout.strip()                      # no JSON line pretending to be a result


def test_product_does_not_import_the_oracle():
    """The oracle is test infrastructure: nothing under the package may import it."""
    pkg = os.path.join(ROOT, "ngraph-python_amd")
    offenders = []
    for base, _, files in os.walk(pkg):
        for name in files:
            if name.endswith(".py"):
                text = open(os.path.join(base, name)).read()
                if "import oracle" in text or "from oracle" in text:
                    offenders.append(os.path.join(base, name))
    assert not offenders, offenders


def test_transformer_fails_loudly_without_a_gpu():
    """No CPU fallback: without a device the backend raises instead of computing elsewhere."""
    code = ("import sys; sys.path[:0] = [%r, %r]\n"
            "import ngraph_hip.transformers as ngt\n"
            "from ngraph_hip.transformers.base import UnsupportedTransformerException\n"
            "from ngraph_hip.runtime import hiplib\n"
            "try:\n"
            "    n = hiplib.device_count()\n"
            "except Exception:\n"
            "    n = 0\n"
            "if n:\n"
            "    print('has-gpu')\n"
            "else:\n"
            "    try:\n"
            "        ngt.make_transformer_factory('hipgpu')()\n"
            "        print('constructed')\n"
            "    except UnsupportedTransformerException as e:\n"
            "        print('raised')\n") % (ROOT, os.path.join(ROOT, "ngraph-python_amd"))
    p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert p.stdout.strip() in ("raised", "has-gpu"), (p.stdout, p.stderr)


def test_user_graphs_of_the_compiled_leg_have_no_built_in_programs():
    """`bench.py --compiled` compares interpreter and run-time compiled kernels: each of its
    graphs must lower, and must have at least one stage the library carries no kernel for
    (else the comparison would measure nothing)."""
    sys.path.insert(0, ROOT)
    import bench
    import ngraph_hip as ng
    import ngraph_hip.transformers as ngt
    from ngraph_hip.runtime import jit
    for name, results, inputs, passes in bench.user_graphs(ng, 512, 1024):
        t = ngt.make_transformer_factory("hipgpu", dry_run=True)()
        try:
            f = t.computation(results, *inputs)
            t.initialize()
            kernels = t.kernel_groups[f].kernels
            for k in kernels:
                k.bind_buffers()
            assert jit.uncovered_programs(kernels, name), name
            assert min(passes.values() if isinstance(passes, dict) else [passes]) >= 2
        finally:
            t.close()


def test_benchmark_workloads_are_the_oracle_configurations():
    """bench.py takes the inputs of its GPU legs from the product tree
    (ngraph_hip/testing/workloads.py) and the oracle only times the CPU leg: both must describe
    the same seeded data."""
    import numpy as np
    sys.path[:0] = [ROOT, os.path.join(ROOT, "ngraph-python_amd")]
    from ngraph_hip.testing import workloads
    from oracle import configs
    for ours, theirs in ((workloads.c1_inputs((64, 33)), configs.c1_inputs((64, 33))),
                         (workloads.c2_inputs(8, 500), configs.c2_inputs(8, 500)),
                         (workloads.c3_inputs(1000), configs.c3_inputs(1000)),
                         (workloads.c4_inputs(16, 8), configs.c4_inputs(16, 8)),
                         (workloads.c5_inputs(4096), configs.c5_inputs(4096))):
        assert len(ours) == len(theirs)
        for a, b in zip(ours, theirs):
            np.testing.assert_array_equal(np.asarray(a), np.asarray(b))


def test_bench_gpu_legs_do_not_touch_the_oracle():
    """Only the CPU-baseline leg of bench.py imports the oracle."""
    text = open(os.path.join(ROOT, "bench.py")).read()
    gpu_legs, cpu_leg = text.split("def cpu_baseline_c2", 1)
    assert "import oracle" not in gpu_legs and "from oracle" not in gpu_legs
    main = cpu_leg.split("def main", 1)[1]
    assert main.index("from oracle import") > main.index("if not args.no_cpu")
