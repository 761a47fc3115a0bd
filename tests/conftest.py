import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG_DIR = os.path.join(ROOT, "cudanative.jl_amd")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_package():
    """Import the package directory `cudanative.jl_amd` under the module name cudanative_jl_amd."""
    name = "cudanative_jl_amd"
    if name in sys.modules:
        return sys.modules[name]
    spec_b = importlib.util.spec_from_file_location("_miw_build", os.path.join(PKG_DIR, "build.py"))
    b = importlib.util.module_from_spec(spec_b)
    spec_b.loader.exec_module(b)
    # The library carries the hash of the sources it was built from.  It is read from the file, not by
    # loading the library: a binary loaded here would stay this process's libmiwmma.so even after a
    # rebuild at the same path, and the tests would then run against the stale kernels.
    if b.built_id() != b.source_id():
        # nothing built yet, or built from other sources: build once (hipcc cross-compiles without a GPU)
        b.build()
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"),
                                                  submodule_search_locations=[PKG_DIR])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    if not os.environ.get("MIWMMA_LIB"):
        loaded = mod._lib.load().miw_build_id().decode()
        if loaded != b.source_id():
            raise RuntimeError("libmiwmma.so in this process has build id %s, the sources have %s" % (loaded, b.source_id()))
    return mod


def pytest_report_header(config):
    try:
        m = load_package()
        return "libmiwmma build id: %s" % m._lib.load().miw_build_id().decode()
    except Exception as e:  # noqa: BLE001
        return "libmiwmma not loadable: %s" % e


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def miw():
    return load_package()


@pytest.fixture(scope="session")
def gpu(miw):
    """Initialised library on device 0.  GPU tests fail (not skip) when the HIP path cannot run."""
    miw.init(0)
    return miw


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle
