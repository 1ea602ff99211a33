import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # the libraries are built beforehand and travel with the tree; build them only if nothing is there
    import importlib.util
    spec = importlib.util.spec_from_file_location("mor_amd_build", os.path.join(ROOT, "mor_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.ensure_built()


@pytest.fixture(scope="session")
def oracle():
    from oracle import mor_oracle
    mor_oracle.lib()
    return mor_oracle
