import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def load_package(name="gradients_c_amd", lib_path=None):
    """Import the product package; its directory name contains a dot, so it is loaded from its path under the
    module name gradients_c_amd.  A second instance under another name can be pointed at another build of the
    same C sources (the host-logic tests use the device-less build of tests/host)."""
    if name in sys.modules:
        return sys.modules[name]
    path = os.path.join(ROOT, "gradients.c_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=[os.path.dirname(path)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    if lib_path is not None:
        mod.LIB_PATH = lib_path
    return mod


@pytest.fixture(scope="session")
def oracle():
    from oracle import gd_oracle
    gd_oracle.lib()
    return gd_oracle


@pytest.fixture(scope="session")
def gda():
    return load_package()


@pytest.fixture(scope="session")
def backend(gda):
    """One HIP backend for the whole GPU session (fails loudly without a device)."""
    be = gda.Backend()
    yield be
    be.close()


@pytest.fixture(scope="session")
def host():
    """The host core, operator front ends and decoder built against the device-less test backend (tests/host):
    the same C sources as the product, no GPU needed.  Returns (package instance, its decoder module)."""
    import importlib
    import subprocess
    host_dir = os.path.join(ROOT, "tests", "host")
    subprocess.run(["make", "-C", host_dir], check=True, capture_output=True)
    pkg = load_package("gradients_c_amd_host", os.path.join(host_dir, "libgradients_host.so"))
    dec = importlib.import_module("gradients_c_amd_host.decoder")
    return pkg, dec
