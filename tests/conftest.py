"""Shared fixtures: loads the hyphenated package directory as `ops_sparse_amd`
and registers the `gpu` marker (tests that need a real MI355X)."""
import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_package():
    """Import ops-sparse_amd/ under the importable name ops_sparse_amd."""
    if "ops_sparse_amd" in sys.modules:
        return sys.modules["ops_sparse_amd"]
    pkg_dir = os.path.join(ROOT, "ops-sparse_amd")
    spec = importlib.util.spec_from_file_location(
        "ops_sparse_amd", os.path.join(pkg_dir, "__init__.py"), submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["ops_sparse_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real AMD MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def osa():
    return load_package()


@pytest.fixture(scope="session")
def workloads(osa):
    import importlib
    return importlib.import_module("ops_sparse_amd.workloads")


@pytest.fixture(scope="session")
def gpu_ctx(osa):
    """(torch device, stream, handle) for GPU tests; the library must be loadable."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    osa.lib()  # raises if libops_sparse.so is missing: there is no fallback to test
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    # torch's own kernels (fills, clones, uploads) go on the same stream as the library's, so the two are ordered
    torch.cuda.set_stream(stream)
    handle = osa.Handle(stream)
    yield dev, stream, handle
    handle.close()
