import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load what is built; only when nothing is built (a fresh checkout) they build it first."""
    lib = os.path.join(ROOT, "tinytorch_amd", "lib")
    built = [os.path.join(lib, "libttsdpa.so"), os.path.join(lib, "libtinytorch_host.so"),
             os.path.join(lib, "test_sdpa_host")]
    if not any(os.path.exists(f) for f in built):
        import __graft_entry__
        __graft_entry__.build()


def load_golden(name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)
    d = {k: z[k] for k in z.files}
    d["causal"] = bool(int(d["causal"]))
    d["scale"] = float(d["scale"]) if "scale" in d else None
    d.setdefault("mask", None)
    return d


def golden_names():
    return sorted(f[:-4] for f in os.listdir(GOLDEN) if f.endswith(".npz"))


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle
    oracle.lib()
    return oracle
