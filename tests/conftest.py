import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "cv-cuda_amd")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def load_package():
    """Imports cv-cuda_amd/ (not a valid identifier) under the module name cvcuda_amd."""
    if "cvcuda_amd" in sys.modules:
        return sys.modules["cvcuda_amd"]
    libdir = os.path.join(PKG, "lib")
    if not (os.path.exists(os.path.join(libdir, "libcvcuda.so")) and os.path.exists(os.path.join(libdir, "libnvcv_types.so"))):
        spec = importlib.util.spec_from_file_location("_cvbuild", os.path.join(PKG, "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    spec = importlib.util.spec_from_file_location("cvcuda_amd", os.path.join(PKG, "__init__.py"),
                                                  submodule_search_locations=[PKG])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["cvcuda_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def load_oracle():
    if "cv_oracle" in sys.modules:
        return sys.modules["cv_oracle"]
    spec = importlib.util.spec_from_file_location("cv_oracle", os.path.join(ROOT, "oracle", "cv_oracle.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules["cv_oracle"] = mod
    spec.loader.exec_module(mod)
    mod.lib()
    return mod


@pytest.fixture(scope="session")
def cv():
    return load_package()


@pytest.fixture(scope="session")
def K(cv):
    return sys.modules["cvcuda_amd._constants"]


@pytest.fixture(scope="session")
def orc():
    return load_oracle()


@pytest.fixture(scope="session")
def gpu(cv):
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    return torch.device("cuda:0")
