"""A request's state between admission and its last token (reference engine/sequence.py:80-136)."""
from __future__ import annotations

from enum import Enum, auto
from itertools import count

from ..sampling.params import SamplingParams


class SequenceStatus(Enum):
    WAITING = auto()     # queued: new, or preempted and to be recomputed
    RUNNING = auto()     # holds a cache row: prompt partly fed, or decoding
    FINISHED = auto()


class Sequence:
    _ids = count()

    def __init__(self, prompt_token_ids: list[int], sampling_params: SamplingParams):
        if not prompt_token_ids:
            raise ValueError("a prompt must hold at least one token")
        self.seq_id = next(Sequence._ids)
        self.prompt_token_ids = [int(t) for t in prompt_token_ids]
        self.completion_token_ids: list[int] = []
        self.token_logprobs: list[float | None] = []
        self.top_logprobs: list[dict | None] = []
        self.sampling_params = sampling_params
        self.status = SequenceStatus.WAITING
        self.num_computed_tokens = 0        # tokens whose keys and values are in the cache
        self.num_preemptions = 0
        self.seed = sampling_params.seed if sampling_params.seed is not None else self.seq_id
        self.sampler_notes: dict = {}       # what the sampler keeps about this request between steps

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_completion_tokens(self) -> int:
        return len(self.completion_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.completion_token_ids)

    @property
    def num_remaining_tokens(self) -> int:
        """Known tokens not yet fed: more than one while a prompt (or a recomputation) is under
        way, exactly one when the last sampled token waits to be fed."""
        return self.num_tokens - self.num_computed_tokens

    @property
    def is_decoding(self) -> bool:
        return self.status is SequenceStatus.RUNNING and self.num_remaining_tokens == 1 and self.num_completion_tokens > 0

    def next_tokens(self, n: int) -> list[int]:
        """The next ``n`` known tokens that are not in the cache yet (no copy of the whole history:
        a decode step of a long request asks for one token)."""
        start, stop = self.num_computed_tokens, self.num_computed_tokens + n
        prompt = len(self.prompt_token_ids)
        if stop <= prompt:
            return self.prompt_token_ids[start:stop]
        if start >= prompt:
            return self.completion_token_ids[start - prompt:stop - prompt]
        return self.prompt_token_ids[start:] + self.completion_token_ids[:stop - prompt]

    def append_token(self, token: int, logprob=None, top=None) -> None:
        self.completion_token_ids.append(int(token))
        self.token_logprobs.append(logprob)
        self.top_logprobs.append(top)

    def tokens_left_to_generate(self) -> int:
        return self.sampling_params.max_tokens - self.num_completion_tokens
