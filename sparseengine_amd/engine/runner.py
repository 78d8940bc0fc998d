"""The model runner: model + cache manager + the one step function.

``step(entries)`` takes a batch of (request, its next tokens, wanted places): portions of prompts
beside single decoded tokens, cut anywhere.  It runs exactly those tokens, as one batch, against
the cache earlier steps left, and returns float32 logits at the wanted places.  Sampling is not
done here.  (The reference's step is ``ModelRunner.run(seqs, is_prefill)``,
engine/model_runner.py:2572-2660: prefill chunks *or* decode tokens, sampled inside.)
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..cache.manager import CacheManager
from ..config.registry import Architecture, read_config_json, resolve_architecture
from ..weights import loader as weight_loader
from ..weights import random_weights
from .batch import BatchBuilder, StepItem

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}") from None


def require_true_float32() -> None:
    """No reduced-precision matrix mode for float32 products of the BLAS library."""
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")


def kernels_for_program(device: str):
    """What the programs (``bin/trace_run``, the command line) hand to the engine they build: ``(kernels,
    device)``.  ``cuda``: ``(None, "cuda")``, the HIP kernels, the only path of the product.  ``cpu`` is a test
    seam of the programs alone: ``SPARSEENGINE_AMD_KERNELS=module:factory`` must then name a stand-in for the
    HIP kernels that works on CPU tensors (the tests' twins, or their host build of the kernel sources); it is
    said so on stderr.  The variable without ``cpu`` is refused, and neither ``ModelRunner`` nor ``LLM`` looks
    at the environment."""
    import importlib
    import os
    import sys
    seam = os.environ.get("SPARSEENGINE_AMD_KERNELS")
    if device != "cpu":
        if seam:
            raise ValueError("SPARSEENGINE_AMD_KERNELS is set, but the device asked for is not cpu: the variable "
                             "replaces the kernels by a stand-in on the CPU (a test seam); unset it")
        return None, device
    if not seam:
        raise ValueError("device cpu needs SPARSEENGINE_AMD_KERNELS=module:factory (a test seam); the engine's "
                         "own kernels run on the GPU only")
    module, _, factory = seam.partition(":")
    print(f"[sparseengine_amd] test seam: the kernels are replaced by {seam} on the CPU", file=sys.stderr, flush=True)
    return getattr(importlib.import_module(module), factory)(), "cpu"


@dataclass
class StepEntry:
    request_id: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)


class ModelRunner:
    def __init__(self, arch: Architecture, cfg, params_factory, *, dtype, device="cuda", kv_page_size=64,
                 num_kvcache_tokens: int | None = None, max_num_seqs: int = 8, max_model_len: int | None = None,
                 mlp_chunk_size: int = 16384, kernels=None, gpu_memory_utilization: float = 0.9, method=None,
                 cache_manager_cls=None, validate_runtime_invariants: bool = False):
        """``method`` / ``cache_manager_cls``: the sparse method's runtime and the class of its cache manager
        (config/method_registry.py); absent: the dense method on the paged cache manager.
        ``validate_runtime_invariants``: before every attention launch the host checks that each block-table
        entry the launch will read names a page of the pool."""
        self.arch, self.model_config = arch, cfg
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        require_true_float32()
        if kernels is None:
            from ..kernels.hip_ops import HipKernels      # raises if there is no GPU or no library
            kernels = HipKernels()
        self.kernels = kernels
        self.spec = arch.build_spec(cfg)
        self.model = arch.make_model(self.spec, chunk_tokens=mlp_chunk_size)
        if getattr(kernels, "libraries", None):
            from ..kernels import library
            library.ensure_built(sorted(self.model.all_kernel_libraries()))
        self.max_model_len = int(max_model_len or self.spec.max_position)
        if self.max_model_len > self.spec.max_position:
            raise ValueError(f"max_model_len {self.max_model_len} exceeds the model's "
                             f"max_position_embeddings {self.spec.max_position}")
        self.model.limit_positions(self.max_model_len)
        decls = self.model.all_param_decls()
        self.params = params_factory(decls, self.dtype, self.device)
        self.model.bind_all(self.params)
        self.model.finalize_all(kernels)
        self.kv_page_size = int(kv_page_size)
        requests = self.model.cache_requests()
        if num_kvcache_tokens is None or int(num_kvcache_tokens) <= 0:
            num_kvcache_tokens = self.derive_cache_tokens(requests, max_num_seqs, gpu_memory_utilization)
        self.cache = (cache_manager_cls or CacheManager)(requests, max_rows=max_num_seqs,
                                                         max_model_len=self.max_model_len, page_size=self.kv_page_size,
                                                         num_tokens=int(num_kvcache_tokens), dtype=self.dtype,
                                                         device=self.device)
        shapes = {}
        if getattr(kernels, "libraries", None):
            for position in requests:
                key = getattr(self.model.layers[self.spec.schedule[position].layer].mixer, "work_key", None)
                if key is not None:
                    shapes.setdefault(self.cache.group_of_position[position], set()).add(key())
        self.builder = BatchBuilder(kernels, self.cache, self.dtype, self.device, self.spec.vocab_size,
                                    attention_shapes=shapes)
        if method is None:
            from ..config.method_registry import PassThroughMethod
            method = PassThroughMethod()
        self.method = method
        method.bind(self.cache)
        self.validate_runtime_invariants = bool(validate_runtime_invariants)

    def derive_cache_tokens(self, requests, max_num_seqs: int, utilization: float) -> int:
        """Tokens of cache that fit the memory left after the weights: ``utilization`` of the card
        minus what is in use, capped by what ``max_num_seqs`` requests of full length could hold."""
        from ..parts.base import PagedKVRequest
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        per_token = sum(2 * r.kv_heads * r.head_dim * itemsize for r in requests.values()
                        if isinstance(r, PagedKVRequest))
        cap = max_num_seqs * self.max_model_len
        if per_token == 0 or self.device.type != "cuda":
            return cap
        free, total = torch.cuda.mem_get_info(self.device)
        usable = free - int((1.0 - utilization) * total) - (2 << 30)      # 2 GiB kept for step buffers
        if usable <= per_token * max([self.kv_page_size] + [r.page_size or 0 for r in requests.values()
                                                            if isinstance(r, PagedKVRequest)]):
            raise RuntimeError("no GPU memory is left for the cache after the weights")
        return min(cap, usable // per_token)

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder: str, **kwargs) -> "ModelRunner":
        raw = read_config_json(folder)
        arch = resolve_architecture(raw)
        cfg = arch.parse_config(raw)

        def factory(decls, dtype, device):
            return weight_loader.load_parameters(folder, arch, cfg, decls, dtype, device)
        return cls(arch, cfg, factory, **kwargs)

    @classmethod
    def from_random(cls, raw_config: dict, seed: int = 0, options: dict | None = None,
                    on_device: bool | None = False, **kwargs) -> "ModelRunner":
        """``on_device``: draw the weights with the device's generator (other values than the
        host's, which a written folder holds); None decides by size: above 2^30 parameters the host
        would take minutes."""
        arch = resolve_architecture(raw_config)
        cfg = arch.parse_config(raw_config)

        def factory(decls, dtype, device):
            dtypes = random_weights.random_parameter_dtypes(arch, cfg, decls, dtype)
            params = weight_loader.allocate_parameters(decls, dtypes, device)
            large = sum(p.numel() for p in params.values()) > 2 ** 30
            draw_there = (large if on_device is None else bool(on_device)) and torch.device(device).type == "cuda"
            random_weights.fill_random(params, arch, cfg, decls, seed, options, on_device=draw_there)
            return params
        return cls(arch, cfg, factory, **kwargs)

    # ------------------------------------------------------------------ requests
    def admit(self, request_id) -> int:
        return self.cache.admit(request_id)

    def release(self, request_id) -> None:
        self.cache.free(request_id)

    def can_step(self, entries) -> bool:
        """Whether the cache has room for these (request_id, new token count) pairs; requests
        not yet admitted are counted with an empty row."""
        need = {g.index: 0 for g in self.cache.groups}
        new_rows = 0
        for request_id, n in entries:
            row = self.cache.row_of(request_id) if self.cache.has_row(request_id) else None
            if row is not None:
                for gi, pages in self.cache.pages_needed(row, n).items():
                    need[gi] += pages
            else:
                new_rows += 1
                for gi, pages in self.cache.pages_for_tokens(n).items():
                    need[gi] += pages
            for gi, pages in self.method.extra_pages(row, n).items():
                need[gi] += pages
        free = self.cache.free_pages()
        return new_rows <= self.cache.num_free_rows and all(need[g] <= free[g] for g in need)

    # ------------------------------------------------------------------ the step
    @torch.no_grad()
    def step(self, entries: list[StepEntry], taps: dict | None = None, forced_routing=None) -> torch.Tensor:
        """Run the entries' tokens as one batch; float32 logits ``[wanted, vocab]`` in the order
        of the entries and of their ``want`` lists.  A request that holds no row yet is admitted.
        If the cache cannot take the step, ``OutOfPages`` is raised and nothing has changed."""
        admitted = []
        try:
            items = []
            for e in entries:
                if not self.cache.has_row(e.request_id):
                    self.cache.admit(e.request_id)
                    admitted.append(e.request_id)
                items.append(StepItem(self.cache.row_of(e.request_id), list(e.tokens), list(e.want)))
            fb = self.builder.build(items)
        except Exception:
            for request_id in admitted:
                self.cache.free(request_id)
            raise
        fb.taps = taps
        fb.forced_routing = forced_routing      # measurement and test seam (parts/feed_forward.py: _force)
        fb.method = self.method
        fb.check_tables = self.validate_runtime_invariants
        self.method.prepare_step(fb)
        logits = self.model.forward(fb)
        self.method.finish_step(fb)
        return logits
