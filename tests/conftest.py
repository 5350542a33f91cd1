import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def load_package():
    """Imports the hyphen-named package directory under the module name torch_xpu_ops_amd."""
    if "torch_xpu_ops_amd" in sys.modules:
        return sys.modules["torch_xpu_ops_amd"]
    pdir = os.path.join(ROOT, "torch-xpu-ops_amd")
    spec = importlib.util.spec_from_file_location(
        "torch_xpu_ops_amd", os.path.join(pdir, "__init__.py"), submodule_search_locations=[pdir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["torch_xpu_ops_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    return load_package()


@pytest.fixture(scope="session")
def cabi(pkg):
    pkg.cabi.lib()  # raises if the kernel library has not been built
    return pkg.cabi


@pytest.fixture(scope="session")
def ops(pkg):
    return pkg.load_host_library()


@pytest.fixture(scope="session")
def oracle():
    import oracle as o
    o.lib()
    return o


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _clear_overrides(request):
    yield
    if "torch_xpu_ops_amd" in sys.modules:
        try:
            sys.modules["torch_xpu_ops_amd"].cabi.clear_overrides()
        except Exception:
            pass
