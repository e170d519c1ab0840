"""A request and its sampling parameters (reference: mercury/request.py:7-96)."""

from __future__ import annotations

import enum
from dataclasses import dataclass, field


class RequestState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    ABORTED = "aborted"


@dataclass
class SamplingParams:
    """temperature <= 0 is greedy; top_p < 1 keeps the nucleus; `seed`, when given, replaces
    the engine's seed for this request's random stream (the reference stores a seed and never
    reads it, mercury/request.py:14-23)."""

    temperature: float = 0.0
    top_p: float = 1.0
    ignore_eos: bool = False
    seed: int | None = None

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0


@dataclass
class Request:
    rid: str
    prompt: list
    max_tokens: int
    arrival: float
    hashes: list
    params: SamplingParams = field(default_factory=SamplingParams)
    session_id: str | None = None

    out: list = field(default_factory=list)
    tokens: list = field(default_factory=list, repr=False)   # prompt + out, kept in step
    num_computed: int = 0        # tokens whose keys and values are in the cache
    num_cached: int = 0          # of those, how many admission found already cached
    state: RequestState = RequestState.WAITING
    admitted_at: float | None = None
    last_admitted_at: float | None = None
    first_token_at: float | None = None
    finished_at: float | None = None
    preemptions: int = 0
    recomputed_tokens: int = 0
    finish_reason: str | None = None

    def __post_init__(self) -> None:
        self.tokens = list(self.prompt) + list(self.out)

    def append(self, token: int) -> None:
        """Take a generated token."""
        self.out.append(token)
        self.tokens.append(token)

    @property
    def seq_len(self) -> int:
        return len(self.tokens)

    @property
    def remaining(self) -> int:
        """Tokens that still have to run before the next token can be sampled."""
        return self.seq_len - self.num_computed

    @property
    def prompt_len(self) -> int:
        return len(self.prompt)

    @property
    def running(self) -> bool:
        return self.state is RequestState.RUNNING

    @property
    def done(self) -> bool:
        return self.state in (RequestState.FINISHED, RequestState.ABORTED)

    def queue_delay(self):
        return None if self.admitted_at is None else self.admitted_at - self.arrival

    def record(self) -> dict:
        return {
            "rid": self.rid,
            "session_id": self.session_id,
            "arrival": self.arrival,
            "admitted_at": self.admitted_at,
            "first_token_at": self.first_token_at,
            "finished_at": self.finished_at,
            "queue_delay": self.queue_delay(),
            "prompt_tokens": len(self.prompt),
            "output_tokens": len(self.out),
            "cached_tokens": self.num_cached,
            "recomputed_tokens": self.recomputed_tokens,
            "preemptions": self.preemptions,
            "finish_reason": self.finish_reason,
            "state": self.state.value,
        }
