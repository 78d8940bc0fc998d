"""Random weights from a configuration and a seed.

Every checkpoint tensor is drawn by name: its generator is seeded with a hash of (seed, tensor
name), so the values do not depend on the order, the device or which other tensors exist.
``write_model_folder`` stores them as a model folder (config.json + model.safetensors) through the
same names the loader reads; ``fill_random`` draws them straight into allocated parameters (for
models too large to pass through a file).  The reference's random mode draws N(0, 0.02) for every
floating parameter from one generator in parameter order (debug/tiny_random.py:181-292).
"""
from __future__ import annotations

import hashlib
import json
import os
import sys
import time

import torch
from safetensors.torch import save_file

from ..config.registry import Architecture, resolve_architecture
from ..weights.loader import _indexed_shape

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def tensor_generator(seed: int, name: str, device=None) -> torch.Generator:
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    generator = torch.Generator(device=device) if device is not None else torch.Generator()
    return generator.manual_seed(int.from_bytes(digest[:8], "little") & (2**63 - 1))


def checkpoint_tensors(arch: Architecture, cfg, decls, seed: int, options: dict | None = None, device=None):
    """Yield (name, tensor in its stored dtype) for every tensor of the architecture's table."""
    options = options or {}
    for src in arch.weight_sources(cfg):
        shape = _indexed_shape(decls[src.param].shape, src.index)
        value = arch.random_tensor(cfg, src.name, shape, tensor_generator(seed, src.name, device), options)
        yield src, value.to(_TORCH_DTYPE[options.get("store_dtype") or arch.stored_dtype(src.name)])


def write_model_folder(folder: str, raw_config: dict, seed: int, options: dict | None = None) -> str:
    """Write ``config.json`` and ``model.safetensors`` for the configuration; returns the folder."""
    arch = resolve_architecture(raw_config)
    cfg = arch.parse_config(raw_config)
    decls = arch.make_model(arch.build_spec(cfg)).all_param_decls()
    os.makedirs(folder, exist_ok=True)
    tensors = {src.name: value.contiguous() for src, value in checkpoint_tensors(arch, cfg, decls, seed, options)}
    weights_file = os.path.join(folder, "model.safetensors")
    save_file(tensors, weights_file)
    umask = os.umask(0)       # the writer leaves the file readable by its owner only: give it the usual mode
    os.umask(umask)
    os.chmod(weights_file, 0o666 & ~umask)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(arch.config_to_dict(cfg), fh, indent=1)
    return folder


def random_parameter_dtypes(arch, cfg, decls, engine_dtype) -> dict[str, torch.dtype]:
    stored = {}
    for src in arch.weight_sources(cfg):
        stored.setdefault(src.param, set()).add(arch.stored_dtype(src.name))
    out = {}
    for path, decl in decls.items():
        if decl.policy == "int32":
            out[path] = torch.int32
        elif decl.policy == "float32" or engine_dtype == torch.float32 or "float32" in stored.get(path, ()):
            out[path] = torch.float32
        else:
            out[path] = engine_dtype
    return out


def fill_random(params: dict[str, torch.Tensor], arch: Architecture, cfg, decls, seed: int,
                options: dict | None = None, on_device: bool = False) -> None:
    """Fill allocated parameters with the same values ``write_model_folder`` would store.

    ``on_device=True`` draws with the device's generator instead (same names and seeds, other
    values than the host's; for sizes where host generation would take minutes)."""
    options = options or {}
    device = next(iter(params.values())).device if on_device else None
    total = sum(p.numel() for p in params.values())
    done, last = 0, time.monotonic()
    for src, value in checkpoint_tensors(arch, cfg, decls, seed, options, device=device):
        target = params[src.param]
        (target[src.index] if src.index else target).copy_(value)
        done += value.numel()
        if time.monotonic() - last > 20:      # a large model takes minutes on the host: say that it moves
            last = time.monotonic()
            print(f"[sparseengine_amd] random weights: {100 * done / total:.0f} % of {total / 1e9:.1f} G values drawn",
                  file=sys.stderr, flush=True)
