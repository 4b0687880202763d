import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure).  Built on demand if absent."""
    import _oracle
    return _oracle.load_oracle()


@pytest.fixture(scope="session")
def ref():
    """Self-contained reference headers compiled as-is (oracle/_ref/libref.so).
    Only exists where it was built from the reference tree; tests that need it skip otherwise."""
    import _oracle
    lib = _oracle.load_ref()
    if lib is None:
        pytest.skip("oracle/_ref/libref.so not built (reference tree not available)")
    return lib


@pytest.fixture(scope="session")
def lib():
    """The product C-ABI library.  Missing library = failure, never a fallback."""
    # The tests use torch for device buffers, and this torch wheel bundles its own HIP/HSA
    # runtime.  A process can drive the GPU through one runtime only: whichever of two is
    # initialised second sees no device.  Loading torch first makes the library bind to the
    # runtime already in the process (same soname) instead of bringing /opt/rocm's.
    import torch  # noqa: F401
    import aws_ofi_nccl_amd as m
    if not os.path.exists(m.LIB_PATH):
        from aws_ofi_nccl_amd import build
        build.build_library()
    return m.load()


@pytest.fixture(scope="session")
def gpu(lib):
    """Initialises the GPU through the C ABI; gpu-marked tests depend on it."""
    import torch
    assert torch.cuda.is_available(), "gpu-marked test started without a GPU"
    rc = lib.ofi_amd_gpu_init()
    assert rc == 0, "ofi_amd_gpu_init failed: %d" % rc
    torch.cuda.init()
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _announce(request):
    # name the case before it touches the GPU, flushed, so a lost box still names it
    if request.node.get_closest_marker("gpu"):
        print("\n[gpu-case] %s" % request.node.nodeid, flush=True)
    yield
