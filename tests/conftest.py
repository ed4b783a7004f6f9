import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.binding import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def oracle64():
    import numpy as np
    from oracle.binding import Oracle
    return Oracle(np.float64)


@pytest.fixture(scope="session")
def reference():
    """The real reference, compiled (oracle/_ref/libdlref.so); absent on hosts
    where oracle/Makefile.ref was never run."""
    from oracle.binding import Reference, reference_available
    if not reference_available():
        pytest.skip("oracle/_ref/libdlref.so not built (needs /root/reference)")
    return Reference()


@pytest.fixture(scope="session")
def golden_leaves():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "leaves.npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def golden_mlp():
    import numpy as np
    return np.load(os.path.join(ROOT, "tests", "golden", "mlp.npz"), allow_pickle=False)


def load_package():
    """Imports deep-learning_amd/ (hyphenated directory) as `deep_learning_amd`."""
    import importlib.util
    if "deep_learning_amd" in sys.modules:
        return sys.modules["deep_learning_amd"]
    pkg_dir = os.path.join(ROOT, "deep-learning_amd")
    spec = importlib.util.spec_from_file_location("deep_learning_amd", os.path.join(pkg_dir, "__init__.py"),
                                                  submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["deep_learning_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def pkg():
    return load_package()


@pytest.fixture(scope="session")
def dl(pkg):
    """A dlmi context on cuda:0.  GPU tests only; never falls back."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    d = pkg.Dlmi(0)
    yield d
    d.close()
