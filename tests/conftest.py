import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_ROOT = os.path.join(ROOT, "ngraph-python_amd")
for p in (ROOT, PKG_ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip_runtime():
    """One device context for the whole GPU test session."""
    from ngraph_hip.runtime import HipRuntime
    rt = HipRuntime(0)
    yield rt
    rt.close()


def default_kernel_choice():
    """False when an environment knob of the library forces another kernel than the planner
    would pick (then tests still check results, but not which kernel produced them)."""
    import os
    return not any(os.environ.get(k) for k in ("NGH_FORCE_INTERP", "NGH_NO_TILES", "NGH_CACHE_POLICY", "NGH_TILE4",
                                                  "NGH_ROW_WAVE_CHUNKS", "NGH_STREAM_MIB", "NGH_NO_RAGGED", "NGH_NO_CHAIN"))
