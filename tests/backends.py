"""Where the tests marked ``gpu`` run their kernels.

``hip`` (the default): the GPU, through the product's own path.  ``emu``: the same kernel sources
built for the host (tests/emu), every tensor argument next to an inaccessible page; chosen with
``SPARSEENGINE_AMD_TEST_BACKEND=emu`` for a whole run, or per test with ``use("emu")``.  The
emulated backend is slow: tests ask ``ACTIVE.slow`` and shorten their workloads.

    SPARSEENGINE_AMD_TEST_BACKEND   hip | emu
    SPARSEENGINE_AMD_EMU_GUARD      after (overruns fault, the default) | before (underruns fault)
    SPARSEENGINE_AMD_EMU_SCHEDULE   ascending | descending | shuffled    order of a block's threads
    SPARSEENGINE_AMD_EMU_LDS        at_wait | at_issue                   when loads into shared memory land
"""
from __future__ import annotations

import contextlib
import os


class Backend:
    name = "hip"
    device = "cuda"
    slow = False

    def kernels(self):
        from sparseengine_amd.kernels.hip_ops import HipKernels
        return HipKernels()

    def runner_kwargs(self) -> dict:
        return {}

    def llm_kwargs(self) -> dict:
        return {}

    def available(self) -> bool:
        import torch
        return torch.cuda.is_available()

    @contextlib.contextmanager
    def session(self):
        yield


class EmulatedBackend(Backend):
    name = "emu"
    device = "cpu"
    slow = True

    def __init__(self, guard=None, schedule=None, lds=None, seed=0):
        self.guard = guard or os.environ.get("SPARSEENGINE_AMD_EMU_GUARD", "after")
        self.schedule = schedule or os.environ.get("SPARSEENGINE_AMD_EMU_SCHEDULE", "ascending")
        self.lds = lds or os.environ.get("SPARSEENGINE_AMD_EMU_LDS", "at_wait")
        self.seed = seed

    def kernels(self):
        from tests.emu.kernels import EmuKernels
        return EmuKernels()

    def runner_kwargs(self) -> dict:
        return dict(device="cpu", kernels=self.kernels())

    def llm_kwargs(self) -> dict:
        return dict(_device="cpu", _kernels=self.kernels())

    def available(self) -> bool:
        from tests.emu import build
        return build.host_compiler() is not None

    @contextlib.contextmanager
    def session(self):
        from tests.emu.kernels import emulated
        with emulated(guard=self.guard, schedule=self.schedule, seed=self.seed, lds=self.lds):
            yield


class TwinBackend(Backend):
    """The tensor-library twins of the kernels on the CPU: the host side of the engine alone."""
    name = "twin"
    device = "cpu"

    def kernels(self):
        from tests.twin_kernels import TwinKernels
        return TwinKernels()

    def runner_kwargs(self) -> dict:
        return dict(device="cpu", kernels=self.kernels())

    def llm_kwargs(self) -> dict:
        return dict(_device="cpu", _kernels=self.kernels())

    def available(self) -> bool:
        return True


def _from_environment() -> Backend:
    name = os.environ.get("SPARSEENGINE_AMD_TEST_BACKEND", "hip")
    if name == "emu":
        return EmulatedBackend()
    if name != "hip":
        raise ValueError(f"SPARSEENGINE_AMD_TEST_BACKEND={name!r}: hip or emu")
    return Backend()


ACTIVE: Backend = _from_environment()


@contextlib.contextmanager
def use(backend):
    """Run the block on another backend (an instance, or "emu" / "hip")."""
    global ACTIVE
    if isinstance(backend, str):
        backend = {"emu": EmulatedBackend, "twin": TwinBackend, "hip": Backend}[backend]()
    saved = ACTIVE
    ACTIVE = backend
    try:
        with backend.session():
            yield backend
    finally:
        ACTIVE = saved
