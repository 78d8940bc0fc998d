import faulthandler
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")
    # A fault on the GPU ends the process from a thread of the runtime.  The stock handler then
    # prints the stack of every thread, which pushes the name of the test out of whatever tail of
    # the output survives; the aborting thread alone is enough.
    faulthandler.enable(file=sys.__stderr__, all_threads=False)


def pytest_collection_modifyitems(config, items):
    from tests import backends
    if backends.ACTIVE.available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process" if backends.ACTIVE.name == "hip"
                            else "no host compiler for the emulated kernels")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _kernel_backend(request):
    """Tests marked ``gpu`` run inside their backend's session (the emulated one routes the kernel
    calls to the host build; the GPU's needs nothing)."""
    from tests import backends
    if "gpu" not in request.keywords:
        yield
        return
    with backends.ACTIVE.session():
        yield


def _on_gpu(item) -> bool:
    return "gpu" in item.keywords and not any(m.name == "skip" for m in item.iter_markers())


@pytest.hookimpl(hookwrapper=True, tryfirst=True)
def pytest_runtest_protocol(item, nextitem):
    """The name of every GPU test goes out, flushed, before the test touches the GPU (and before
    output is captured for it): if the process dies under it, the last name printed is the test
    that was running."""
    if _on_gpu(item):
        for stream in (sys.__stdout__, sys.__stderr__):
            try:
                stream.write(f"\n[test] {item.nodeid}\n")
                stream.flush()
            except (OSError, ValueError):
                pass
    yield


@pytest.hookimpl(trylast=True)
def pytest_runtest_teardown(item, nextitem):
    """Kernels run asynchronously; waiting for them here pins a failure to the test that made it."""
    if _on_gpu(item):
        import torch
        from tests import backends
        if backends.ACTIVE.name == "hip" and torch.cuda.is_available():
            torch.cuda.synchronize()
