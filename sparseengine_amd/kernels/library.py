"""Building and loading the HIP kernel libraries.

Every ``csrc/<name>.hip`` becomes one shared library ``csrc/lib/<name>.<digest>.so`` built with
``hipcc`` for gfx950; the digest covers the source, the shared header and the flags, so a stale
library is never loaded.  Libraries are looked up in the source tree first and in a per-user
cache folder second (for a read-only checkout); what is missing is compiled on first use, in
parallel, with a progress line every few seconds.  There is no fallback: a library that cannot
be found or built raises ``KernelLibraryError``.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
OFFLOAD_ARCH = "gfx950"
# packed float instructions are switched off for the device pass (the host pass does not know
# the feature and says so; that is harmless)
HIPCC_FLAGS = [
    "-O3", f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-std=c++17", "-Wno-pass-failed",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Per source.  The attention kernels keep their accumulators in ordinary vector registers: left to
# itself the compiler parks them in the accumulation registers and copies all of them to and fro
# in every step of the key loop, which costs more instructions than the step's own arithmetic.
EXTRA_FLAGS = {
    "attention_mfma": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def _flags(name: str) -> list[str]:
    return HIPCC_FLAGS + EXTRA_FLAGS.get(name, [])


class KernelLibraryError(RuntimeError):
    pass


def _digest(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(_flags(name)).encode())
    for path in [CSRC / f"{name}.hip"] + sorted(CSRC.glob("*.h")):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return h.hexdigest()[:16]


def _user_cache_dir() -> Path:
    root = os.environ.get("SPARSEENGINE_AMD_CACHE")
    if root:
        return Path(root)
    return Path(tempfile.gettempdir()) / f"sparseengine_amd_{os.getuid()}"


def _candidate_dirs() -> list[Path]:
    return [CSRC / "lib", _user_cache_dir()]


def library_path(name: str) -> Path | None:
    """The built library of ``name`` that matches the current source, if there is one."""
    file_name = f"{name}.{_digest(name)}.so"
    for folder in _candidate_dirs():
        path = folder / file_name
        if path.is_file():
            return path
    return None


def _writable_dir() -> Path:
    for folder in _candidate_dirs():
        try:
            folder.mkdir(parents=True, exist_ok=True)
            probe = folder / f".probe_{os.getpid()}"
            probe.write_bytes(b"")
            probe.unlink()
            return folder
        except OSError:
            continue
    raise KernelLibraryError("no writable folder for the kernel libraries: tried " +
                             ", ".join(str(d) for d in _candidate_dirs()))


def available_sources() -> list[str]:
    return sorted(p.stem for p in CSRC.glob("*.hip"))


def build(names=None, force: bool = False, verbose: bool = True) -> dict[str, Path]:
    """Compile the named libraries (all by default) that are missing, or all of them if ``force``."""
    names = list(names) if names is not None else available_sources()
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    result: dict[str, Path] = {}
    jobs = []
    out_dir = None
    for name in names:
        if not (CSRC / f"{name}.hip").is_file():
            raise KernelLibraryError(f"no kernel source csrc/{name}.hip")
        existing = None if force else library_path(name)
        if existing is not None:
            result[name] = existing
            continue
        if not os.path.exists(hipcc):
            raise KernelLibraryError(
                f"kernel library '{name}' is not built and hipcc was not found; run "
                "`python -c 'import __graft_entry__ as g; g.build()'` where hipcc is installed")
        out_dir = out_dir or _writable_dir()
        target = out_dir / f"{name}.{_digest(name)}.so"
        partial = out_dir / f".{name}.{os.getpid()}.tmp.so"
        cmd = [hipcc, *_flags(name), "-o", str(partial), str(CSRC / f"{name}.hip")]
        proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        jobs.append((name, proc, partial, target))
    if jobs and verbose:
        print(f"[sparseengine_amd] compiling {len(jobs)} kernel librar"
              f"{'y' if len(jobs) == 1 else 'ies'} for {OFFLOAD_ARCH}: "
              + ", ".join(j[0] for j in jobs), file=sys.stderr, flush=True)
    start = last = time.time()
    pending = list(jobs)
    while pending:
        still = []
        for job in pending:
            name, proc, partial, target = job
            if proc.poll() is None:
                still.append(job)
                continue
            output = proc.stdout.read()
            if proc.returncode != 0 or not partial.is_file():
                for other in pending:
                    if other[1].poll() is None:
                        other[1].kill()
                raise KernelLibraryError(f"hipcc failed for csrc/{name}.hip:\n{output}")
            for old in target.parent.glob(f"{name}.*.so"):
                if old != target:
                    try:
                        old.unlink()
                    except OSError:
                        pass
            os.replace(partial, target)
            result[name] = target
        pending = still
        if pending:
            time.sleep(0.2)
            if verbose and time.time() - last > 5:
                last = time.time()
                print(f"[sparseengine_amd] still compiling ({int(last - start)} s): "
                      + ", ".join(j[0] for j in pending), file=sys.stderr, flush=True)
    if jobs and verbose:
        print(f"[sparseengine_amd] kernels built in {time.time() - start:.1f} s",
              file=sys.stderr, flush=True)
    return result


_loaded: dict[str, ctypes.CDLL] = {}


def load(name: str) -> ctypes.CDLL:
    """The loaded library ``name``; built first if it is missing."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    path = library_path(name) or build([name])[name]
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as exc:
        raise KernelLibraryError(f"cannot load kernel library {path}: {exc}") from exc
    _loaded[name] = lib
    return lib


def ensure_built(names) -> None:
    """Build, in one parallel batch, whichever of ``names`` is missing."""
    missing = [n for n in dict.fromkeys(names) if library_path(n) is None]
    if missing:
        build(missing)
