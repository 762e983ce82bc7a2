import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_PARENT = os.path.join(ROOT, "qfactory-ae_amd")
for p in (ROOT, PKG_PARENT):
    if p not in sys.path:
        sys.path.insert(0, p)

# Specialisations are prebuilt into the in-tree cache by __graft_entry__.build(); a miss compiles
# with hipcc on the spot.
os.environ.setdefault("QFACTORY_CACHE_DIR", os.path.join(PKG_PARENT, "jit_cache"))
os.environ.setdefault("QFACTORY_LOG_LEVEL", "WARNING")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import qf_oracle
    qf_oracle.build()
    return qf_oracle
