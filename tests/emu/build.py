"""Builds the kernel sources of ``sparseengine_amd/csrc`` for the host (tests only).

A source is copied with three kinds of edits and compiled with the host clang against
``hip_emu.h``: ``kernel<<<grid, block, shared, stream>>>(args)`` becomes a call of the emulator's
launcher, ``extern __shared__`` arrays become pointers to the emulated dynamic shared memory, and the
few inline-assembly statements become calls of their emulated meaning.  Everything else (indexing,
masks, clamps, reductions, the order of synchronisation) is the text the GPU compiler sees.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import tempfile
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE.parent.parent / "sparseengine_amd" / "csrc"
SOURCES = ("norm", "rope_kv", "attention_generic", "attention_mfma", "moe", "moe_mfma", "sampling")
FLAGS = ["-O2", "-g", "-std=c++17", "-shared", "-fPIC", "-x", "c++", "-Wno-unknown-pragmas", "-Wno-pass-failed",
         "-Wno-unused-value", "-Wno-gnu-designator", "-fno-strict-aliasing"]


class EmulatorBuildError(RuntimeError):
    pass


def host_compiler() -> str | None:
    for candidate in ("/opt/rocm/llvm/bin/clang++", shutil.which("clang++")):
        if candidate and os.path.exists(candidate):
            return candidate
    return None


# ------------------------------------------------------------------------------------- the edits
_ASM = [
    (r'asm\("v_max_f32 %0, %1, %2" : "=v"\(r\) : "v"\(a\), "v"\(b\)\);', "r = emu_max_bare(a, b);"),
    (r'asm\("v_max3_f32 %0, %1, %2, %3" : "=v"\(r\) : "v"\(a\), "v"\(b\), "v"\(c\)\);', "r = emu_max3_bare(a, b, c);"),
    # keeps values in registers before a loop: nothing to do on the host
    (r'asm volatile\("" : "\+v"\([^;]*\);', ";"),
    # wait states after matrix instructions: nothing to do on the host
    (r'asm volatile\("s_nop 15\\n\\ts_nop 15" : "\+v"\([^;]*\);', ";"),
    (r'asm volatile\("s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %1, off"\s*:\s*:[^;]*;',
     "emu_load16_to_lds(src, lds_addr);"),
    (r'asm volatile\("s_mov_b32 m0, %0\\n\\ts_nop 0\\n\\tglobal_load_lds_dwordx4 %1, %2"\s*:\s*:[^;]*;',
     "emu_load16_to_lds(static_cast<const char*>(base) + offset, lds_addr);"),
]
_DYNAMIC_SHARED = re.compile(
    r"extern\s+__shared__\s+(?:__align__\(\d+\)\s+)?((?:unsigned\s+)?\w+)\s+(\w+)\[\];")


def _matching(text: str, start: int, open_ch: str, close_ch: str) -> int:
    """Index just past the bracket that closes the one at ``start``."""
    depth = 0
    for i in range(start, len(text)):
        if text[i] == open_ch:
            depth += 1
        elif text[i] == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
    raise EmulatorBuildError("unbalanced brackets near: " + text[start:start + 80])


def _split_top_level(text: str) -> list[str]:
    parts, depth, current = [], 0, []
    for ch in text:
        if ch in "([{<":
            depth += 1
        elif ch in ")]}>":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append("".join(current).strip())
            current = []
        else:
            current.append(ch)
    parts.append("".join(current).strip())
    return parts


def _rewrite_launches(text: str) -> str:
    out, cursor = [], 0
    while True:
        at = text.find("<<<", cursor)
        if at < 0:
            out.append(text[cursor:])
            return "".join(out)
        # the kernel expression before <<<: an identifier with optional template arguments
        begin = at
        while begin > 0 and text[begin - 1].isspace():
            begin -= 1
        if text[begin - 1] == ">":
            depth, i = 0, begin - 1
            while i >= 0:
                if text[i] == ">":
                    depth += 1
                elif text[i] == "<":
                    depth -= 1
                    if depth == 0:
                        break
                i -= 1
            begin = i
        while begin > 0 and (text[begin - 1].isalnum() or text[begin - 1] in "_:"):
            begin -= 1
        kernel = text[begin:at].strip()
        close = text.find(">>>", at)
        config = _split_top_level(text[at + 3:close])
        if not 2 <= len(config) <= 4:
            raise EmulatorBuildError(f"launch configuration of {kernel}: {config}")
        args_open = close + 3
        while text[args_open].isspace() or text[args_open] == "\\":
            args_open += 1
        if text[args_open] != "(":
            raise EmulatorBuildError(f"no argument list after the launch of {kernel}")
        args_close = _matching(text, args_open, "(", ")")
        name = re.match(r"[\w:]+", kernel).group(0)
        shared = config[2] if len(config) > 2 else "0"
        out.append(text[cursor:begin])
        out.append(f'emu_launch("{name}", {config[0]}, {config[1]}, {shared}, [&] {{ {kernel}{text[args_open:args_close]}; }})')
        cursor = args_close


def transform(text: str) -> str:
    text = text.replace("#include <hip/hip_runtime.h>", '#include "hip_emu.h"')
    for pattern, replacement in _ASM:
        text = re.sub(pattern, replacement, text, flags=re.S)
    left = re.search(r"\basm\s*(?:volatile\s*)?\((?!\"\" ::: \"memory\"\)).{0,80}", text, flags=re.S)
    if left:      # a compiler barrier is the only statement that stays as it is
        raise EmulatorBuildError("an inline-assembly statement has no emulation: " + left.group(0))
    text = _DYNAMIC_SHARED.sub(lambda m: f"{m.group(1)}* {m.group(2)} = static_cast<{m.group(1)}*>(emu_dynamic_shared());", text)
    return _rewrite_launches(text)


# ------------------------------------------------------------------------------------- building
def _digest() -> str:
    h = hashlib.sha256()
    for path in sorted(CSRC.glob("*.h")) + [CSRC / f"{n}.hip" for n in SOURCES] + sorted(HERE.glob("*.h")) + \
            sorted(HERE.glob("*.cpp")) + [Path(__file__)]:
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:16]


def build_dir() -> Path:
    root = os.environ.get("SPARSEENGINE_AMD_EMU_CACHE") or os.path.join(tempfile.gettempdir(),
                                                                        f"sparseengine_amd_emu_{os.getuid()}")
    return Path(root) / _digest()


def build(verbose: bool = False) -> Path:
    """Compile the runtime and every kernel library that is missing; returns their folder."""
    out = build_dir()
    wanted = ["emu_rt"] + list(SOURCES)
    if all((out / f"{n}.so").is_file() for n in wanted):
        return out
    compiler = host_compiler()
    if compiler is None:
        raise EmulatorBuildError("no host clang++ (the emulated build needs ext_vector_type and __bf16)")
    out.mkdir(parents=True, exist_ok=True)
    shutil.copy(HERE / "hip_emu.h", out / "hip_emu.h")
    for header in CSRC.glob("*.h"):
        (out / header.name).write_text(transform(header.read_text()))
    jobs = []
    for name in wanted:
        if (out / f"{name}.so").is_file():
            continue
        if name == "emu_rt":
            source = HERE / "emu_rt.cpp"
        else:
            source = out / f"{name}.cpp"
            source.write_text(transform((CSRC / f"{name}.hip").read_text()))
        partial = out / f".{name}.{os.getpid()}.so"
        cmd = [compiler, *FLAGS, f"-I{out}", "-o", str(partial), str(source)]
        jobs.append((name, partial, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for name, partial, proc in jobs:
        output, _ = proc.communicate()
        if proc.returncode != 0:
            raise EmulatorBuildError(f"host build of {name} failed:\n{output[-6000:]}")
        if verbose and output.strip():
            print(output)
        os.replace(partial, out / f"{name}.so")
    return out


_loaded: dict[str, ctypes.CDLL] = {}


def load(name: str) -> ctypes.CDLL:
    if name not in _loaded:
        folder = build()
        if "emu_rt" not in _loaded:      # first and globally: the kernel libraries link against it at load time
            _loaded["emu_rt"] = ctypes.CDLL(str(folder / "emu_rt.so"), mode=ctypes.RTLD_GLOBAL)
        if name != "emu_rt":
            _loaded[name] = ctypes.CDLL(str(folder / f"{name}.so"))
    return _loaded[name]
