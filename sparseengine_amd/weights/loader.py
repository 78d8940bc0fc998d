"""Weights from safetensors, by tensor name.

The loader reads the headers of every ``*.safetensors`` file of a model folder, checks them
against the architecture's table (tensor name -> parameter and slice) and against the shapes the
parts declare, and reports everything that is wrong in ONE error: missing tensors, unexpected
tensors, wrong shapes, duplicates across files, quantised tensors.  Only then are parameters
allocated and filled.  Tensors are kept in bfloat16 (or upcast for a float32 engine); a tensor
the file stores in 32-bit float stays float32, integer tables become int32.

Reference behaviour this follows: files sorted, at least one (utils/loader.py:687-688);
duplicate key across shards is an error (:750-755); q/k/v rows stacked into one matrix
(layers/linear.py:453-468); expert w1/w3 stacked as [gate; up] (operators/moe.py:147-222);
unknown names are errors, the M2 class ignores nothing (utils/loader.py:243-245,873).
"""
from __future__ import annotations

import os
from dataclasses import dataclass

import torch
from safetensors import safe_open

from ..config.registry import Architecture, WeightSource
from ..parts.base import ParamDecl

_FLOAT32_NAMES = {"F32", "F64"}
_HALF_NAMES = {"BF16", "F16"}
_INT_NAMES = {"I8", "I16", "I32", "I64", "U8", "BOOL"}


class WeightLoadError(ValueError):
    """All problems of a checkpoint at once: ``missing``, ``unexpected``, ``wrong_shape``, ``other``."""

    def __init__(self, folder, missing, unexpected, wrong_shape, other):
        self.missing, self.unexpected, self.wrong_shape, self.other = missing, unexpected, wrong_shape, other
        lines = [f"cannot load weights from {folder}:"]

        def section(title, entries):
            if entries:
                shown = entries[:12]
                lines.append(f"  {title} ({len(entries)}): " + ", ".join(shown)
                             + (f", ... and {len(entries) - len(shown)} more" if len(entries) > len(shown) else ""))
        section("missing tensors", missing)
        section("unexpected tensors", unexpected)
        section("wrong shapes", wrong_shape)
        section("other problems", other)
        super().__init__("\n".join(lines))


@dataclass
class StoredTensor:
    file: str
    shape: tuple[int, ...]
    dtype: str            # the safetensors dtype name


def index_checkpoint(folder: str):
    """name -> StoredTensor over all safetensors files; (index, duplicate names)."""
    files = sorted(f for f in os.listdir(folder) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{folder} holds no .safetensors file")
    index: dict[str, StoredTensor] = {}
    duplicates = []
    for file in files:
        with safe_open(os.path.join(folder, file), framework="pt") as fh:
            for name in fh.keys():
                sl = fh.get_slice(name)
                if name in index:
                    duplicates.append(f"{name} (in {index[name].file} and {file})")
                    continue
                index[name] = StoredTensor(file, tuple(sl.get_shape()), str(sl.get_dtype()))
    return index, duplicates


def _indexed_shape(shape, index) -> tuple[int, ...]:
    out = []
    for dim, size in enumerate(shape):
        if dim < len(index):
            ix = index[dim]
            if isinstance(ix, int):
                continue
            start, stop, _ = ix.indices(size)
            out.append(max(0, stop - start))
        else:
            out.append(size)
    return tuple(out)


def plan_dtypes(decls: dict[str, ParamDecl], sources: list[WeightSource], index, engine_dtype):
    """Storage dtype of every parameter: see ``ParamDecl``."""
    stored: dict[str, set] = {}
    for src in sources:
        if src.name in index:
            stored.setdefault(src.param, set()).add(index[src.name].dtype)
    out = {}
    for path, decl in decls.items():
        kinds = stored.get(path, set())
        if decl.policy == "int32" or (kinds and kinds <= _INT_NAMES):
            out[path] = torch.int32
        elif decl.policy == "float32" or engine_dtype == torch.float32 or kinds & _FLOAT32_NAMES:
            out[path] = torch.float32
        else:
            out[path] = engine_dtype
    return out


def check_checkpoint(folder, arch: Architecture, cfg, decls: dict[str, ParamDecl]):
    """Raise ``WeightLoadError`` listing every problem, or return (index, sources)."""
    index, duplicates = index_checkpoint(folder)
    sources = arch.weight_sources(cfg)
    missing, unexpected, wrong, other = [], [], [], [f"duplicate tensor {d}" for d in duplicates]
    expected = {}
    for src in sources:
        if src.name in expected:
            other.append(f"table names {src.name} twice")
        expected[src.name] = src
        if src.param not in decls:
            other.append(f"{src.name} targets the unknown parameter {src.param}")
    quantised = sorted(n for n, t in index.items()
                       if t.dtype.startswith("F8") or n.endswith("weight_scale_inv") or n.endswith("weight_scale"))
    if quantised:
        other.append(f"quantised checkpoints are not supported ({len(quantised)} FP8/scale tensors, "
                     f"e.g. {quantised[0]})")
    for name, src in expected.items():
        if name not in index:
            missing.append(name)
            continue
        if src.param not in decls:
            continue
        want = _indexed_shape(decls[src.param].shape, src.index)
        if index[name].shape != want:
            wrong.append(f"{name}: stored {list(index[name].shape)}, expected {list(want)}")
    for name in index:
        if name not in expected and not arch.ignored_tensor(name) and name not in quantised:
            unexpected.append(name)
    covered = {src.param for src in sources}
    for path in decls:
        if path not in covered:
            other.append(f"no checkpoint tensor fills the parameter {path}")
    if missing or unexpected or wrong or other:
        raise WeightLoadError(folder, sorted(missing), sorted(unexpected), wrong, other)
    return index, sources


def allocate_parameters(decls, dtypes, device) -> dict[str, torch.Tensor]:
    return {path: torch.empty(decl.shape, dtype=dtypes[path], device=device) for path, decl in decls.items()}


def fill_parameters(folder, params: dict[str, torch.Tensor], index, sources) -> None:
    by_file: dict[str, list[WeightSource]] = {}
    for src in sources:
        by_file.setdefault(index[src.name].file, []).append(src)
    for file, file_sources in sorted(by_file.items()):
        with safe_open(os.path.join(folder, file), framework="pt") as fh:
            for src in file_sources:
                target = params[src.param]
                view = target[src.index] if src.index else target
                view.copy_(fh.get_tensor(src.name))     # casts to the parameter's dtype


def load_parameters(folder, arch: Architecture, cfg, decls, engine_dtype, device):
    """Check, allocate, fill.  Returns path -> tensor."""
    index, sources = check_checkpoint(folder, arch, cfg, decls)
    dtypes = plan_dtypes(decls, sources, index, engine_dtype)
    params = allocate_parameters(decls, dtypes, device)
    fill_parameters(folder, params, index, sources)
    return params
