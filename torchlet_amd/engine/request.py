"""Per-request state (after /root/reference/src/torchlet/v10_triton_paged_gqa/request.py:7-24)."""
from __future__ import annotations

import itertools
from dataclasses import dataclass, field
from enum import Enum

_ids = itertools.count()


class RequestState(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass(eq=False)          # a request is itself: lists of requests are searched by identity, not by field values
class Request:
    prompt_tokens: list[int]
    max_new_tokens: int = 128
    temperature: float = 0.0
    seed: int = 0
    stop_token_ids: frozenset = frozenset()
    prompt: str = ""
    req_id: str = field(default_factory=lambda: f"req-{next(_ids)}")
    output_tokens: list[int] = field(default_factory=list)
    output: str = ""
    error: Exception | None = None
    computed_tokens: int = 0           # tokens of prompt + output that are in the cache
    state: RequestState = RequestState.WAITING
    finish_reason: str | None = None   # "stop" | "length" | "error"
    preemptions: int = 0

    @property
    def sequence_length(self) -> int:
        return len(self.prompt_tokens) + len(self.output_tokens)

    def tokens(self, start: int, count: int) -> list[int]:
        """``count`` tokens of prompt + output from ``start``."""
        p = len(self.prompt_tokens)
        end = start + count
        if end <= p:
            return self.prompt_tokens[start:end]
        if start >= p:
            return self.output_tokens[start - p:end - p]
        return self.prompt_tokens[start:] + self.output_tokens[:end - p]
