"""The typed runtime configuration.  Its fields are exactly the keyword arguments of
``LLM(model, **kwargs)``; an unknown keyword is an error.  Names and meanings are the reference's
where it has them (configs/runtime.py:51-105, configs/groups.py, configs/scheduling.py:15-186);
``dtype``, ``kv_page_size``, ``sampler_seed`` and ``tiny_random_on_device`` are this engine's own.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, fields

from .method_registry import normalize_sparse_method, resolve_prefill_schedule_policy
from .registry import read_config_json, resolve_architecture

AUTO = "auto"
AUTO_TOKEN_BUDGET = 65536     # upper end of the automatic per-step token budget


@dataclass
class Config:
    model: str
    max_num_batched_tokens: int | str = AUTO      # token budget of one step
    max_num_seqs_in_batch: int = 32               # requests in one step
    max_model_len: int | None = None              # None: the model's max_position_embeddings
    max_decoding_seqs: int | None = None          # None: max_num_seqs_in_batch
    max_num_seqs_in_gpu: int | None = None        # rows of the cache; None: max(3 * batch, decoding)
    engine_prefill_chunk_size: int | str | None = AUTO   # largest prompt portion; auto: the budget
    prefill_schedule_policy: str = AUTO
    decode_reservation_tokens: int = 1024         # room kept per decoding request when admitting prompts
    mlp_chunk_size: int = 16384
    gpu_memory_utilization: float = 0.9
    num_kvcache_slots: int = -1                   # tokens of cache; -1: derived from free memory
    sparse_method: str = ""
    tensor_parallel_size: int = 1
    expert_parallel_size: int = 1
    data_parallel_size: int = 1
    tiny_random: bool = False                     # random weights for the folder's config.json
    tiny_random_config: str | None = None         # JSON (text or file) of config.json overrides
    tiny_random_seed: int = 0
    tiny_random_on_device: bool | None = None     # draw with the device's generator; None: above 2^30 parameters
    eos: int = -1
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    enable_profiler: bool = False
    validate_runtime_invariants: bool = False
    throughput_log_interval_s: float = 0.0
    dtype: str = "bfloat16"                       # "bfloat16" | "float32"
    kv_page_size: int = 64
    sampler_seed: int = 0
    # derived, not keyword arguments
    raw_model_config: dict = field(default=None, init=False, repr=False)
    model_config: object = field(default=None, init=False, repr=False)
    architecture: object = field(default=None, init=False, repr=False)

    @classmethod
    def keyword_names(cls) -> set[str]:
        return {f.name for f in fields(cls) if f.init}

    @classmethod
    def from_kwargs(cls, model: str, **kwargs) -> "Config":
        unknown = sorted(set(kwargs) - cls.keyword_names())
        if unknown:
            raise ValueError(f"unknown configuration keys {unknown}; known: {sorted(cls.keyword_names())}")
        return cls(model, **kwargs)

    def __post_init__(self):
        for name in ("tensor_parallel_size", "expert_parallel_size", "data_parallel_size"):
            if getattr(self, name) != 1:
                raise ValueError(f"{name} must be 1: this engine runs on one GPU")
        self.sparse_method = normalize_sparse_method(self.sparse_method)
        self.prefill_schedule_policy = resolve_prefill_schedule_policy(self.sparse_method, self.prefill_schedule_policy)
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.kv_page_size <= 0 or self.kv_page_size % 8:
            raise ValueError(f"kv_page_size must be a positive multiple of 8, got {self.kv_page_size}")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ValueError("gpu_memory_utilization must be in (0, 1]")
        if self.max_num_seqs_in_batch <= 0:
            raise ValueError("max_num_seqs_in_batch must be positive")
        if self.mlp_chunk_size <= 0:
            raise ValueError("mlp_chunk_size must be positive")
        if self.decode_reservation_tokens < 0:
            raise ValueError("decode_reservation_tokens must not be negative")
        self.eos_token_ids = tuple(int(t) for t in (self.eos_token_ids or ()))

        raw = dict(read_config_json(self.model))
        if self.tiny_random_config:
            if not self.tiny_random:
                raise ValueError("tiny_random_config needs tiny_random=True")
            text = self.tiny_random_config
            if os.path.isfile(text):
                with open(text) as fh:
                    text = fh.read()
            overrides = json.loads(text)
            unknown = sorted(k for k in overrides if k not in raw)
            if unknown:
                raise ValueError(f"tiny_random_config overrides keys that config.json does not have: {unknown}")
            raw.update(overrides)
        self.raw_model_config = raw
        self.architecture = resolve_architecture(raw)
        self.model_config = self.architecture.parse_config(raw)
        model_len = int(self.architecture.build_spec(self.model_config).max_position)
        if self.max_model_len is None:
            self.max_model_len = model_len
        elif not 0 < self.max_model_len <= model_len:
            raise ValueError(f"max_model_len must be in (0, {model_len}], got {self.max_model_len}")

        if self.max_decoding_seqs is None:
            self.max_decoding_seqs = self.max_num_seqs_in_batch
        if self.max_decoding_seqs <= 0:
            raise ValueError("max_decoding_seqs must be positive")
        if self.max_num_seqs_in_gpu is None:
            self.max_num_seqs_in_gpu = max(3 * self.max_num_seqs_in_batch, self.max_decoding_seqs)
        if self.max_num_seqs_in_gpu < self.max_decoding_seqs:
            raise ValueError("max_num_seqs_in_gpu must be at least max_decoding_seqs")
        if self.max_num_batched_tokens == AUTO:
            self.max_num_batched_tokens = min(AUTO_TOKEN_BUDGET, max(self.max_model_len, self.max_decoding_seqs))
        if int(self.max_num_batched_tokens) < self.max_decoding_seqs:
            raise ValueError("max_num_batched_tokens must be at least max_decoding_seqs")
        self.max_num_batched_tokens = int(self.max_num_batched_tokens)
        if self.engine_prefill_chunk_size in (AUTO, None):
            self.engine_prefill_chunk_size = self.max_num_batched_tokens
        self.engine_prefill_chunk_size = int(self.engine_prefill_chunk_size)
        if self.engine_prefill_chunk_size <= 0:
            raise ValueError("engine_prefill_chunk_size must be positive")
