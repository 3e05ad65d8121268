import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_built():
    """Load what is built; compile only if nothing is there."""
    pkg = os.path.join(ROOT, "optimized_transducer_amd")
    if not (os.path.exists(os.path.join(pkg, "libot_transducer.so"))
            and os.path.exists(os.path.join(pkg, "_optimized_transducer.so"))):
        # the build script by path, so that the package is first imported once its extension exists
        import importlib.util
        spec = importlib.util.spec_from_file_location("_ot_build", os.path.join(pkg, "build.py"))
        build = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(build)
        build.build_all()
    from oracle import oracle
    oracle.build()


_ensure_built()


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)
