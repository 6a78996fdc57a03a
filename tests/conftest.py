import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("rex-sc_amd", "oracle", ""):
    p = os.path.join(ROOT, sub) if sub else ROOT
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import json
    import numpy as np
    path = os.path.join(ROOT, "tests", "golden", "ref_cpu_ext.npz")
    data = np.load(path, allow_pickle=False)
    meta = json.loads(bytes(data["meta"]).decode())
    return data, meta


@pytest.fixture(scope="session", autouse=True)
def _oracle_built():
    """The oracle is compiled by __graft_entry__.build(); build it on demand for a bare checkout."""
    so = os.path.join(ROOT, "oracle", "_build", "librexsc_oracle.so")
    if not os.path.exists(so):
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import build as oracle_build
        oracle_build.build_oracle()
