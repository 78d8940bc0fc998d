"""The engine's kernel interface served by the host build of the kernel sources (tests only).

``EmuKernels`` is ``HipKernels`` with CPU tensors: the same Python shape checks, the same entry
points, the same kernel text (see ``build.py`` and ``hip_emu.h``).  Every tensor that goes to an entry
point is first copied into memory that ends right before an inaccessible page (``guard="after"``)
or begins right after one (``guard="before"``), and copied back afterwards: a kernel that reads or
writes outside a tensor ends the process with a message that names the call, the kernel, the block,
the thread and the tensor.  Tensors of one call that share memory (an output that is its input, a
view of a wider row) stay together in one such copy.
"""
from __future__ import annotations

import contextlib
import ctypes

import torch

from sparseengine_amd.kernels import hip_ops

from . import build


class _Arg:
    """A tensor on its way into an entry point (what ``hip_ops._ptr`` gives in emulated mode)."""
    __slots__ = ("tensor",)

    def __init__(self, tensor: torch.Tensor):
        self.tensor = tensor


def _span(t: torch.Tensor) -> tuple[int, int]:
    """First and one-past-last byte address the view can touch."""
    if t.numel() == 0:
        return t.data_ptr(), t.data_ptr()
    last = sum((size - 1) * stride for size, stride in zip(t.shape, t.stride()))
    return t.data_ptr(), t.data_ptr() + (last + 1) * t.element_size()


class _Settings:
    guard = "after"          # where the inaccessible page lies: "after" (overruns), "before" (underruns), None
    poison_outputs = False


settings = _Settings()


class _EmuFunction:
    def __init__(self, lib_name: str, fn_name: str):
        lib = build.load(lib_name)
        self.rt = build.load("emu_rt")
        self.rt.emu_rt_guarded.restype = ctypes.c_void_p
        self.rt.emu_rt_guarded.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_size_t]
        self.rt.emu_rt_release.argtypes = [ctypes.c_void_p]
        self.rt.emu_rt_label.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        self.rt.emu_rt_call.argtypes = [ctypes.c_char_p]
        self.fn = getattr(lib, fn_name)
        self.fn.argtypes = hip_ops._SIGNATURES[lib_name][fn_name]
        self.fn.restype = ctypes.c_int
        self.name = fn_name

    def __call__(self, *args):
        self.rt.emu_rt_call(self.name.encode())
        if settings.guard is None:
            return self.fn(*[a.tensor.data_ptr() if isinstance(a, _Arg) else a for a in args])
        # tensors whose byte ranges overlap stay together
        spans = []           # [begin, end, [argument indices]]
        for index, a in enumerate(args):
            if not isinstance(a, _Arg):
                continue
            begin, end = _span(a.tensor)
            merged = [begin, end, [index]]
            rest = []
            for s in spans:
                if s[0] < merged[1] and merged[0] < s[1] or (s[0] == merged[0] and s[1] == merged[1]):
                    merged = [min(s[0], merged[0]), max(s[1], merged[1]), s[2] + merged[2]]
                else:
                    rest.append(s)
            spans = rest + [merged]
        call_args = list(args)
        copies = []
        for begin, end, indices in spans:
            size = end - begin
            guarded = self.rt.emu_rt_guarded(max(size, 1), int(settings.guard == "before"), begin)
            if not guarded:
                raise MemoryError("no guarded memory")
            self.rt.emu_rt_label(guarded, f"argument {'/'.join(str(i) for i in indices)} of {self.name}".encode())
            if size:
                ctypes.memmove(guarded, begin, size)
            copies.append((guarded, begin, size))
            for i in indices:
                call_args[i] = guarded + (args[i].tensor.data_ptr() - begin)
        try:
            status = self.fn(*call_args)
        finally:
            for guarded, begin, size in copies:
                if size:
                    ctypes.memmove(begin, guarded, size)
                self.rt.emu_rt_release(guarded)
        return status


class _EmuFunctions:
    def __init__(self):
        self._cache = {}

    def get(self, lib_name: str, fn_name: str):
        key = (lib_name, fn_name)
        if key not in self._cache:
            self._cache[key] = _EmuFunction(lib_name, fn_name)
        return self._cache[key]


@contextlib.contextmanager
def emulated(guard: str | None = "after", schedule: str = "ascending", seed: int = 0, lds: str = "at_wait"):
    """Route ``hip_ops`` to the host build for the duration of the block."""
    modes = {"ascending": 0, "descending": 1, "shuffled": 2}
    rt = build.load("emu_rt")
    rt.emu_rt_schedule.argtypes = [ctypes.c_int, ctypes.c_uint]
    rt.emu_rt_schedule(modes[schedule], seed)
    rt.emu_rt_set_lds_mode({"at_wait": 0, "at_issue": 1}[lds])
    saved = (hip_ops._fn, hip_ops._ptr, hip_ops._stream, settings.guard)
    hip_ops._fn = _EmuFunctions()
    hip_ops._ptr = lambda t: None if t is None else _Arg(t)
    hip_ops._stream = lambda: None
    settings.guard = guard
    try:
        yield
    finally:
        hip_ops._fn, hip_ops._ptr, hip_ops._stream, settings.guard = saved
        rt.emu_rt_schedule(0, 0)
        rt.emu_rt_set_lds_mode(0)


class EmuKernels(hip_ops.HipKernels):
    """``HipKernels`` without the GPU: use inside ``emulated()``."""

    def __init__(self):
        self._attention_partials = None
        self._sample_partials = None


class EmulatedProgramKernels(EmuKernels):
    """For a program that names its kernels through ``SPARSEENGINE_AMD_KERNELS``: the emulated
    session (settings from the environment, see tests/backends.py) stays open until the process ends."""
    _session = None

    def __init__(self):
        super().__init__()
        if EmulatedProgramKernels._session is None:
            import os
            EmulatedProgramKernels._session = emulated(
                guard=os.environ.get("SPARSEENGINE_AMD_EMU_GUARD", "after"),
                schedule=os.environ.get("SPARSEENGINE_AMD_EMU_SCHEDULE", "ascending"),
                lds=os.environ.get("SPARSEENGINE_AMD_EMU_LDS", "at_wait"))
            EmulatedProgramKernels._session.__enter__()
