"""One request inside the engine: its tokens, sampling settings and what it holds of the cache
(reference atomserve/sequence.py:17-115, without the draft-model fields).

    WAITING --admit--> RUNNING --EOS / max_tokens / abort--> FINISHED
       ^                  |
       +----preempt-------+      (cache given back; recomputed when readmitted)

Only the scheduler changes a sequence; the step function reads it.
"""

from dataclasses import dataclass, field
from enum import Enum
from typing import Optional

from atomserve_amd.cache.manager import RequestCache


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 is greedy; top_k 0 disables it; top_p keeps the smallest set whose mass
    reaches p; presence_penalty is subtracted from the logits of tokens already generated;
    seed fixes the request's random stream (reference atomserve/sequence.py:23-43)."""

    temperature: float = 0.6
    top_k: int = 20
    top_p: float = 0.95
    presence_penalty: float = 0.0
    max_tokens: int = 4096
    seed: Optional[int] = None
    ignore_eos: bool = False

    def validated(self) -> "SamplingParams":
        """Itself, or a ValueError that names the setting outside its range."""
        if not self.temperature >= 0:
            raise ValueError(f"temperature must be 0 (greedy) or positive, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be 0 (all tokens) or positive, got {self.top_k}")
        if not 0 < self.top_p <= 1:
            raise ValueError(f"top_p must lie in (0, 1], got {self.top_p}")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        return self


# The model card's settings for its two modes (reference atomserve/sequence.py:46-48).
THINKING_PARAMS = SamplingParams(temperature=0.6, top_p=0.95, top_k=20)
NON_THINKING_PARAMS = SamplingParams(temperature=0.7, top_p=0.8, top_k=20)


@dataclass(eq=False)
class Sequence:
    id: int
    token_ids: list
    params: SamplingParams = field(default_factory=SamplingParams)
    num_prompt_tokens: int = -1
    num_computed_tokens: int = 0  # leading tokens whose cache entries are valid
    cache: RequestCache = None  # pages per group and state slot; set by the scheduler
    num_cached_tokens: int = 0  # prompt tokens found in the prefix cache on admission
    status: SequenceStatus = SequenceStatus.WAITING
    finish_reason: Optional[str] = None  # "stop", "length" or "abort"
    noise_seed: int = 0  # seed of the request's random stream (its own, or drawn by the engine)

    def __post_init__(self) -> None:
        if self.num_prompt_tokens < 0:
            self.num_prompt_tokens = len(self.token_ids)
        if self.cache is None:
            self.cache = RequestCache(tables=[])
        if self.params.seed is not None:
            self.noise_seed = int(self.params.seed)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def output_ids(self) -> list:
        """A copy of the generated tokens; `num_output_tokens` counts them without one."""
        return self.token_ids[self.num_prompt_tokens :]

    def reaches_end(self, num_new_tokens: int) -> bool:
        """Whether computing `num_new_tokens` more covers every known token: only then is
        there a next token to predict (reference atomserve/sequence.py:93-100)."""
        return self.num_computed_tokens + num_new_tokens == len(self.token_ids)


@dataclass
class StepResult:
    """What one step did for one scheduled sequence: new tokens (none for a prompt portion
    that stops short) and how many leading tokens are now in the cache."""

    tokens: list
    num_computed: int
