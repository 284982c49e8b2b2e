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
